/* Hooks of libdragon_hip.so that exist for tests, not for the operator path.
 * Nothing a Dragon operator calls is declared here; a process that serves
 * traffic has no reason to include this header. */
#ifndef DRAGON_HIP_TESTING_H_
#define DRAGON_HIP_TESTING_H_

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference. Clears the count behind
 * dragon_hip_exchange_timed_out (dragon_hip.h) on the current device and sets
 * how many polls, of about a microsecond each, a workgroup of the single-read
 * kernels waits for its peers in launches made afterwards; 0 = the default
 * (about a second). With a patience of 1 nearly every slice gives up and is
 * finished by the repair launch: that is how the tests drive the repair path.
 * The setting is process-wide (every later launch from any thread reads it, and
 * a graph captured while it is set keeps it), and the call clears the counter
 * with a synchronous copy on the null stream: do not call it while other
 * threads launch. Results are correct under any patience; a small one only
 * makes every repaired slice be read twice. */
void dragon_hip_exchange_reset(unsigned patience);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* DRAGON_HIP_TESTING_H_ */
