// NCHW GroupNorm forward for groups that one workgroup of 256, 512 or 1024 threads
// holds whole (up to sixteen packets per thread of 1024: 256 KB in 16-bit types).
//
// A group (n, g) is a contiguous run of D * S elements. Thread t keeps packets
// t, t + kThreads, ... of the group in registers between the statistics and the
// normalisation, so x is read once. Two to seven workgroups share a compute
// unit, by the packets a thread holds, and a workgroup requests
// its next group's packets inside the store loop, slot by slot into the
// registers each store frees, so that the workgroups of a compute unit overlap
// their loads, reductions and stores. The channel of a packet does not depend on
// the group, and the scale (gamma * rsig) and shift (beta) of the group's D
// channels wait in LDS: parameter loads inside the store loop would sit in the
// same in-order queue as the packets requested ahead, and a wait for them would
// be a wait for those packets.
#pragma once

#include "common.h"
#include "sample_slices.h"  // wave_total

namespace dragon_hip {

constexpr int kItemPackets = 16;      // packets per thread at most
constexpr uint32_t kMaxItemChannels = 1024;  // channels per group whose parameters fit the LDS table

// Wavefronts per SIMD asked of the compiler: four (128 registers) hold sixteen packets per
// thread; ten packets fit the 80 registers of six, i.e. three 512-thread workgroups per compute
// unit instead of two (groups of 80 KB in bf16: 58.0 us against 65.2 us).
constexpr int item_waves_per_simd(int vpt) { return vpt == 10 ? 6 : vpt == 12 ? 5 : 4; }

template <typename T, int kVPT, int kThreads>
__global__ __launch_bounds__(kThreads, item_waves_per_simd(kVPT)) void group_norm_forward_items(
    const uint32_t rows, const uint32_t npackets, const uint32_t G, const uint32_t D,
    const uint32_t pps /* packets per channel */, const typename IO<T>::Acc eps,
    const T* __restrict__ x, const typename IO<T>::Acc* __restrict__ gamma,
    const typename IO<T>::Acc* __restrict__ beta, typename IO<T>::Acc* __restrict__ mu,
    typename IO<T>::Acc* __restrict__ rsig, T* __restrict__ y) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kWaves = kThreads / kWaveSize;
  // (every table twice: a group uses the half of its parity, so that the barriers of the
  // group between two uses of a half separate them)
  __shared__ A sums[2][2][kWaves];
  __shared__ A scale[2][kMaxItemChannels], shift[2][kMaxItemChannels];
  const uint32_t t = threadIdx.x;
  const uint32_t wave = t / kWaveSize;
  const A inv_l = A(1) / A(static_cast<int64_t>(npackets) * kVec);
  const size_t L = static_cast<size_t>(npackets) * kVec;
  // the channel (inside the group) of the thread's first packet, and how it advances per slot
  const uint32_t ch0 = t / pps, rem0 = t - ch0 * pps;
  const uint32_t step_ch = kThreads / pps, step_rem = kThreads - step_ch * pps;

  u32x4 raw[kVPT];
  uint32_t row = blockIdx.x;
  {
    const T* in = x + static_cast<size_t>(row < rows ? row : 0u) * L;
    int room = static_cast<int>(npackets) - static_cast<int>(t);
    uint32_t off = t * kVec;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      raw[i] = load_packet(in + (room > 0 ? off : 0u));
      room -= kThreads, off += kThreads * kVec;
      asm volatile("" : "+v"(room), "+v"(off));
    }
  }
  uint32_t half = 0;
  for (; row < rows; row += gridDim.x, half ^= 1u) {
    const bool more = row + gridDim.x < rows;  // uniform over the workgroup
    const size_t base = static_cast<size_t>(row) * L;
    const size_t nbase = static_cast<size_t>(more ? row + gridDim.x : row) * L;
    // the group's parameters: requested now, used after the statistics
    const uint32_t c0 = (row % G) * D;
    A gam = A(0), bet = A(0);
    if (t < D) gam = gamma[c0 + t], bet = beta[c0 + t];

    A s = A(0);
    int room = static_cast<int>(npackets) - static_cast<int>(t);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (room > 0) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) s += v[e];
      }
      room -= kThreads;
      asm volatile("" : "+v"(room));
    }
    s = wave_total(s);
    if ((t & (kWaveSize - 1)) == 0) sums[half][0][wave] = s;
    __syncthreads();
    s = A(0);
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s += sums[half][0][w];
    const A mean = s * inv_l;
    // (the packets are converted again in each pass instead of keeping every converted element)
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
    A q = A(0);
    room = static_cast<int>(npackets) - static_cast<int>(t);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (room > 0) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A d = v[e] - mean;
          q += d * d;
        }
      }
      room -= kThreads;
      asm volatile("" : "+v"(room));
    }
    q = wave_total(q);
    if ((t & (kWaveSize - 1)) == 0) sums[half][1][wave] = q;
    __syncthreads();
    q = A(0);
#pragma unroll
    for (int w = 0; w < kWaves; ++w) q += sums[half][1][w];
    const A rs = acc_rsqrt_exact(q * inv_l + eps);
    if (t == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    if (t < D) scale[half][t] = gam * rs, shift[half][t] = bet;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
    room = static_cast<int>(npackets) - static_cast<int>(t);
    uint32_t off = t * kVec, ch = ch0, rem = rem0;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const bool has = room > 0;
      if (has) {
        const A g = scale[half][ch], b = shift[half][ch];
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = (v[e] - mean) * g + b;
        store_packet(y + base + off, IO<T>::pack(v));
      }
      if (more) raw[i] = load_packet(x + nbase + (has ? off : 0u));
      room -= kThreads, off += kThreads * kVec;
      ch += step_ch, rem += step_rem;
      if (rem >= pps) rem -= pps, ++ch;
      asm volatile("" : "+v"(room), "+v"(off), "+v"(ch), "+v"(rem));
    }
  }
}

struct GroupItemPlan {
  bool ok;
  int threads, vpt;
};

// Groups of whole packets with channels of whole packets that 256 threads hold at
// ten packets per thread, or 512 or 1024 threads at sixteen.
template <typename T>
inline GroupItemPlan plan_group_items(int64_t D, int64_t S) {
  constexpr int kVec = IO<T>::kVec;
  GroupItemPlan p{false, 0, 0};
  if (sizeof(T) > 4 || S % kVec != 0 || D > static_cast<int64_t>(kMaxItemChannels)) return p;
  const int64_t npackets = D * S / kVec;
  // smaller groups stay with the row kernels, which hold several per workgroup
  // (groups of 16 KB in 16-bit types: 45.6 us there against 50.5 us here)
  if (npackets < 256 * 8) return p;
  // The fewest packets per thread that hold the group, on 256 threads where ten packets do: the
  // fewer registers, the more workgroups share a compute unit (seven at eight packets and six at
  // ten on 256 threads; three, three, two and two at eight, ten, twelve and sixteen on 512), and
  // what counts is the bytes they keep in flight together. Measured cold on MI355X, bf16, groups
  // of 40 / 64 / 80 / 96 KB, the chosen flavour against sixteen packets on the smallest workgroup
  // that holds the group: 59.5 / 46.9 / 58.1 / 52.2 us against 61.7 / 50.6 / 63.2 / 53.5 us.
  struct Choice { int vpt, threads; };
  // Beyond 128 KB (in 16-bit types) one 1024-thread workgroup per compute unit: still ahead of
  // cutting the group into slices that exchange their sums (bf16 groups of 147 / 160 / 196 KB:
  // 54.9 / 122 / 54.5 us against 65.4 / 145 / 68.8 us; level at 256 KB).
  constexpr Choice kChoices[] = {{8, 256},  {10, 256}, {8, 512},   {10, 512},  {12, 512},
                                 {16, 512}, {10, 1024}, {12, 1024}, {16, 1024}};
  for (const Choice& c : kChoices) {
    if (npackets > static_cast<int64_t>(c.threads) * c.vpt || D > c.threads) continue;
    p.ok = true;
    p.threads = c.threads;
    p.vpt = c.vpt;
    return p;
  }
  return p;
}

template <typename T>
int try_group_norm_forward_items(int64_t N, int64_t G, int64_t D, int64_t S, float eps,
                                 const void* x, const void* gamma, const void* beta, void* mu,
                                 void* rsig, void* y, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  if constexpr (sizeof(T) > 4) {
    return kNotApplicable;
  } else {
    constexpr int kVec = IO<T>::kVec;
    const GroupItemPlan p = plan_group_items<T>(D, S);
    const int64_t rows = N * G;
    if (!p.ok || !aligned16(x) || !aligned16(y) || rows > 0x7fffffff) return kNotApplicable;
    // A workgroup per group, handed out by the hardware as workgroups finish, keeps the memory
    // system busier than resident workgroups that walk the groups and request one ahead, except
    // for the 512-thread flavours with nearly every slot filled and fewer than four groups per
    // resident workgroup (bf16, 2048 groups of 64 KB: 46.9 us walking against 49.2 us; 8192 groups
    // of 40 KB on 256 threads: 238 us walking against 220 us). Measured cold on MI355X.
    const int64_t npackets = D * S / kVec;
#define LAUNCH(VPT, THREADS)                                                                      \
  {                                                                                               \
    auto kernel = group_norm_forward_items<T, VPT, THREADS>;                                      \
    const unsigned resident = resident_grid(kernel, THREADS, 0);                                  \
    /* (decided on the three or two workgroups per compute unit the flavour is built for, so  */  \
    /* that the choice does not depend on what the occupancy query answers)                   */  \
    const int64_t nominal = static_cast<int64_t>(num_cus()) * (VPT <= 10 ? 3 : 2);                \
    const bool walk = THREADS == 512 && npackets * 4 > static_cast<int64_t>(THREADS) * VPT * 3 && \
        rows < nominal * 4;                                                                       \
    note_flavour("group_norm_forward_items<" #VPT "," #THREADS ">");                              \
    note_number("walk", walk ? 1 : 0);                                                            \
    /* (a launch holds fewer than 2^32 threads: beyond 2^21 workgroups they walk as well) */      \
    const unsigned most = walk ? resident : 1u << 21;                                             \
    hipLaunchKernelGGL(kernel, dim3(rows > most ? most : static_cast<unsigned>(rows)),            \
                       dim3(THREADS), 0, stream, static_cast<uint32_t>(rows),                     \
                       static_cast<uint32_t>(D * S / kVec), static_cast<uint32_t>(G),             \
                       static_cast<uint32_t>(D), static_cast<uint32_t>(S / kVec), A(eps),         \
                       static_cast<const T*>(x), static_cast<const A*>(gamma),                    \
                       static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig),   \
                       static_cast<T*>(y));                                                       \
  }
    if (p.threads == 256) {
      if (p.vpt == 8) LAUNCH(8, 256) else LAUNCH(10, 256)
    } else if (p.threads == 512) {
      if (p.vpt == 8) LAUNCH(8, 512) else if (p.vpt == 10) LAUNCH(10, 512)
      else if (p.vpt == 12) LAUNCH(12, 512) else LAUNCH(16, 512)
    } else {
      if (p.vpt == 10) LAUNCH(10, 1024) else if (p.vpt == 12) LAUNCH(12, 1024) else LAUNCH(16, 1024)
    }
#undef LAUNCH
    return status_of_launch();
  }
}

}  // namespace dragon_hip
