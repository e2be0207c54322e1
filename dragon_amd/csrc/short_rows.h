// Short rows (up to 1024 elements) of any width and alignment, e.g. the
// 197-key attention rows of a vision transformer or 64-wide per-head
// normalisations. A workgroup takes a run of consecutive rows, i.e. one
// contiguous byte range: it copies the aligned 16-byte packets that cover the
// range into LDS, works on the rows there with kL lanes per row (kE elements
// per lane, so short rows do not idle most of a wavefront), and writes the
// range back in aligned packets; only the first and last packet of a range are
// touched element by element. HBM therefore sees aligned, fully coalesced
// 128-bit accesses whatever the row length.
//
// The arithmetic is a policy Op (lane l of a row's group owns the elements
// e = l + j * kL, j < kE):
//   kIn                    staged input tensors (1 or 2)
//   fill0(), fill1()       what the lanes past the row hold
//   begin<kL>(l, C)        per-thread setup (e.g. the parameters of its elements)
//   kSideWords, fetch_side(row, w)   per-row scalars the rows need (e.g. a saved
//                          mean): kSideWords accumulator-typed words per row,
//                          copied into LDS beside the range before the row loop
//   row<kL>(r, side, l, C, v0, v1)   one row (side = its scalars): overwrites v0
//                          with the outputs; all kL lanes of the group enter
//                          together, so it may reduce over them with
//                          group_allreduce<kL>
//   end<kL>(lds, C)        after the workgroup's last row, entered by all threads
//                          (e.g. column sums kept per thread); kEndBytes of LDS
#pragma once

#include <type_traits>

#include "common.h"

namespace dragon_hip {

constexpr int kShortThreads = 256;

// All-reduce over groups of kL adjacent lanes (kL a power of two, 4 .. 64).
template <int kL, typename Op>
__device__ __forceinline__ float group_allreduce(float v, Op op) {
  v = dpp_step<0xB1>(v, op);                              // quad_perm [1,0,3,2]
  v = dpp_step<0x4E>(v, op);                              // quad_perm [2,3,0,1]
  if constexpr (kL >= 8) v = dpp_step<0x141>(v, op);      // row_half_mirror
  if constexpr (kL >= 16) v = dpp_step<0x140>(v, op);     // row_mirror
  if constexpr (kL >= 32) v = op(v, __shfl_xor(v, 16, kWaveSize));
  if constexpr (kL >= 64) v = op(v, __shfl_xor(v, 32, kWaveSize));
  return v;
}
template <int kL, typename Op>
__device__ __forceinline__ double group_allreduce(double v, Op op) {
#pragma unroll
  for (int o = kL / 2; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, kWaveSize));
  return v;
}

// The byte range [a0, a1) of a tensor that starts at `base` and has `total`
// bytes, staged in LDS from the aligned packet that contains a0 on.
struct StagedRange {
  uintptr_t base, total;  // the whole tensor
  uintptr_t a0, a1;       // this range (absolute addresses)
  uintptr_t first;        // a0 rounded down to 16 bytes
  uint32_t packets;       // aligned packets covering the range
  __device__ __forceinline__ StagedRange(const void* tensor, size_t total_bytes, size_t b0,
                                         size_t b1) {
    base = reinterpret_cast<uintptr_t>(tensor), total = total_bytes;
    a0 = base + b0, a1 = base + b1;
    first = a0 & ~static_cast<uintptr_t>(15);
    packets = static_cast<uint32_t>((a1 - first + 15) / 16);
  }
  __device__ __forceinline__ uint32_t lead() const { return static_cast<uint32_t>(a0 - first); }
};

// Packets a thread requests before it waits for the first of them.
constexpr int kStageBatch = 4;

// One packet of `r` that may reach outside the tensor (only the tensor's first
// or last can): read element by element; what lies outside reads as zero.
template <typename T>
__device__ __forceinline__ void stage_in_edge(const StagedRange& r, u32x4* stage, uint32_t p) {
  const uintptr_t addr = r.first + 16u * p;
  T* out = reinterpret_cast<T*>(stage + p);
#pragma unroll
  for (uint32_t i = 0; i < 16 / sizeof(T); ++i) {
    const uintptr_t ea = addr + i * sizeof(T);
    T zero{};
    out[i] = (ea >= r.base && ea + sizeof(T) <= r.base + r.total)
                 ? *reinterpret_cast<const T*>(ea) : zero;
  }
}

// Copies the packets of the ranges into stage0 / stage1 [0 .. r.packets); the
// two ranges (kIn == 2) cover the same bytes of two congruent tensors. A thread
// requests a batch of packets of every tensor before it waits for the first and
// moves them to LDS: the loads of a workgroup travel together instead of one per
// thread at a time. The conditions around the loads are uniform over the
// workgroup. kStream: the tensors are read once and not again soon
// (non-temporal loads).
template <typename T, bool kStream, int kIn>
__device__ __forceinline__ void stage_in(const StagedRange& r0, u32x4* stage0,
                                         const StagedRange& r1, u32x4* stage1) {
  // packets [lo, hi) lie inside the tensor
  const bool head_out = r0.first < r0.base;
  const bool tail_out = r0.first + 16u * static_cast<uintptr_t>(r0.packets) > r0.base + r0.total;
  const uint32_t lo = head_out ? 1u : 0u;
  const uint32_t hi = r0.packets - (tail_out ? 1u : 0u);
  for (uint32_t p0 = lo; p0 < hi; p0 += kShortThreads * kStageBatch) {
    u32x4 v0[kStageBatch], v1[kStageBatch];
#pragma unroll
    for (int k = 0; k < kStageBatch; ++k) {
      if (p0 + k * kShortThreads < hi) {  // uniform
        const uint32_t want = p0 + k * kShortThreads + threadIdx.x;
        const uint32_t p = want < hi ? want : hi - 1;
        const T* a0 = reinterpret_cast<const T*>(r0.first + 16u * static_cast<uintptr_t>(p));
        v0[k] = kStream ? load_packet(a0) : load_packet_keep(a0);
        if constexpr (kIn == 2) {
          const T* a1 = reinterpret_cast<const T*>(r1.first + 16u * static_cast<uintptr_t>(p));
          v1[k] = kStream ? load_packet(a1) : load_packet_keep(a1);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kStageBatch; ++k) {
      const uint32_t p = p0 + k * kShortThreads + threadIdx.x;
      if (p < hi) {
        stage0[p] = v0[k];
        if constexpr (kIn == 2) stage1[p] = v1[k];
      }
    }
  }
  if (head_out && threadIdx.x == 0) {
    stage_in_edge<T>(r0, stage0, 0);
    if constexpr (kIn == 2) stage_in_edge<T>(r1, stage1, 0);
  }
  if (tail_out && threadIdx.x == kWaveSize && !(head_out && r0.packets == 1)) {
    stage_in_edge<T>(r0, stage0, r0.packets - 1);
    if constexpr (kIn == 2) stage_in_edge<T>(r1, stage1, r0.packets - 1);
  }
}

// Writes stage[0 .. r.packets) back to the range `r` of the output: packets
// inside the range whole, the range's first and last packet element by element
// (their other elements belong to neighbouring rows of other workgroups).
template <typename T>
__device__ __forceinline__ void stage_out(const StagedRange& r, const u32x4* stage) {
  for (uint32_t p = threadIdx.x; p < r.packets; p += kShortThreads) {
    const uintptr_t addr = r.first + 16u * p;
    if (addr >= r.a0 && addr + 16 <= r.a1) {
      store_packet(reinterpret_cast<T*>(addr), stage[p]);
    } else {
      const T* in = reinterpret_cast<const T*>(stage + p);
#pragma unroll
      for (uint32_t i = 0; i < 16 / sizeof(T); ++i) {
        const uintptr_t ea = addr + i * sizeof(T);
        if (ea >= r.a0 && ea + sizeof(T) <= r.a1) *reinterpret_cast<T*>(ea) = in[i];
      }
    }
  }
}

// An Op that declares `static constexpr bool kReadOnly = true` only reads its
// rows (a reduction per row): nothing is written back and `out` is not used.
template <typename Op, typename = void>
struct OpReadOnly : std::false_type {};
template <typename Op>
struct OpReadOnly<Op, std::void_t<decltype(Op::kReadOnly)>> : std::bool_constant<Op::kReadOnly> {};

// An Op with a member `set_packed(bool)` accepts the packed element order: when
// a row is exactly kL * kE elements and the tensors are 16-byte aligned, lane l
// owns the contiguous elements l * kE + j instead of l + j * kL and moves them
// with 128-bit LDS accesses. A wavefront then touches one contiguous stretch of
// LDS per access, free of bank conflicts; in the interleaved order its narrow
// accesses hit rows a power of two apart (four- to eight-way conflicts for rows
// of 64 elements). The kernel tells the Op which order is in force before
// begin(); Ops that index per-element parameters must follow it.
// Such an Op also says for which lane counts it wants the order:
// `template <int kL> static constexpr bool packed_ok()`.
template <typename Op, int kL, typename = void>
struct OpPacked : std::false_type {};
template <typename Op, int kL>
struct OpPacked<Op, kL, std::void_t<decltype(Op::template packed_ok<kL>())>>
    : std::bool_constant<Op::template packed_ok<kL>()> {};

// in0, in1 (when kIn == 2) and out must be congruent modulo 16 bytes (they
// usually are: allocations are aligned far beyond that), so that the staged
// packets map one to one. Several workgroups share a compute unit and overlap
// each other's waits; requesting a workgroup's next range ahead into registers
// was measured and is slower (0.59 against 0.73 of the HBM peak for fp16 rows
// of 128).
template <typename T, int kL, int kE, typename Op>
__global__ __launch_bounds__(kShortThreads) void short_rows(
    const int64_t N, const int C, const uint32_t rows_per_chunk, const uint32_t stage_packets,
    const T* in0, const T* in1, T* out, Op op) {
  using A = typename IO<T>::Acc;
  extern __shared__ u32x4 stage[];
  u32x4* stage1 = stage + stage_packets;
  A* side = reinterpret_cast<A*>(stage + stage_packets * Op::kIn);  // per-row scalars of the range
  const size_t row_bytes = static_cast<size_t>(C) * sizeof(T);
  const size_t total = static_cast<size_t>(N) * row_bytes;
  const int l = threadIdx.x % kL;
  const int sub = threadIdx.x / kL;
  constexpr int kRowsPerPass = kShortThreads / kL;
  constexpr int kSide = Op::kSideWords > 0 ? Op::kSideWords : 1;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kLanePackets = kE / kVec;
  bool packed = false;
  if constexpr (OpPacked<Op, kL>::value) {
    packed = C == kL * kE &&
        ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    op.set_packed(packed);
  }
  op.template begin<kL>(l, C);
  for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * rows_per_chunk; row0 < N;
       row0 += static_cast<int64_t>(gridDim.x) * rows_per_chunk) {
    const int rows = static_cast<int>(N - row0 < rows_per_chunk ? N - row0 : rows_per_chunk);
    const StagedRange r0(in0, total, row0 * row_bytes, (row0 + rows) * row_bytes);
    if constexpr (Op::kSideWords > 0) {
      // first, so that these loads travel with the packets'
      A w[kSide];
      for (int i = threadIdx.x; i < rows; i += kShortThreads) {
        op.fetch_side(row0 + i, w);
#pragma unroll
        for (int q = 0; q < kSide; ++q) side[i * kSide + q] = w[q];
      }
    }
    const StagedRange r1(Op::kIn == 2 ? in1 : in0, total, row0 * row_bytes,
                         (row0 + rows) * row_bytes);
    stage_in<T, !OpReadOnly<Op>::value, Op::kIn>(r0, stage, r1, stage1);
    __syncthreads();
    T* tile0 = reinterpret_cast<T*>(reinterpret_cast<char*>(stage) + r0.lead());
    const T* tile1 = reinterpret_cast<const T*>(reinterpret_cast<const char*>(stage1) + r0.lead());
    for (int r = sub; r < rows; r += kRowsPerPass) {
      T* p0 = tile0 + static_cast<size_t>(r) * C;
      const T* p1 = tile1 + static_cast<size_t>(r) * C;
      A v0[kE], v1[kE];
      if (OpPacked<Op, kL>::value && packed) {  // uniform over the grid; rows start on packets
        u32x4* q0 = reinterpret_cast<u32x4*>(p0) + l * kLanePackets;
        const u32x4* q1 = reinterpret_cast<const u32x4*>(p1) + l * kLanePackets;
#pragma unroll
        for (int k = 0; k < kLanePackets; ++k) {
          A t[kVec];
          IO<T>::unpack(q0[k], t);
#pragma unroll
          for (int i = 0; i < kVec; ++i) v0[k * kVec + i] = t[i];
          if constexpr (Op::kIn == 2) {
            IO<T>::unpack(q1[k], t);
#pragma unroll
            for (int i = 0; i < kVec; ++i) v1[k * kVec + i] = t[i];
          }
        }
        op.template row<kL>(row0 + r, side + r * kSide, l, C, v0, v1);
        if constexpr (!OpReadOnly<Op>::value) {
#pragma unroll
          for (int k = 0; k < kLanePackets; ++k) {
            A t[kVec];
#pragma unroll
            for (int i = 0; i < kVec; ++i) t[i] = v0[k * kVec + i];
            q0[k] = IO<T>::pack(t);
          }
        }
        continue;
      }
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const int e = l + j * kL;
        v0[j] = e < C ? IO<T>::load1(p0 + e) : op.fill0();
        if constexpr (Op::kIn == 2) v1[j] = e < C ? IO<T>::load1(p1 + e) : op.fill1();
      }
      op.template row<kL>(row0 + r, side + r * kSide, l, C, v0, v1);
      if constexpr (!OpReadOnly<Op>::value) {
#pragma unroll
        for (int j = 0; j < kE; ++j) {
          const int e = l + j * kL;
          if (e < C) IO<T>::store1(p0 + e, v0[j]);
        }
      }
    }
    __syncthreads();
    if constexpr (!OpReadOnly<Op>::value) {
      const StagedRange ro(out, total, row0 * row_bytes, (row0 + rows) * row_bytes);
      stage_out<T>(ro, stage);
      __syncthreads();  // the stage is refilled by the next range
    }
  }
  op.template end<kL>(reinterpret_cast<A*>(stage), C);
}

struct ShortPlan {
  int lanes, per_lane;
  uint32_t rows_per_chunk, stage_packets;
};
// The stage holds a range of up to 256 * packets_per_thread packets (4 KB per
// unit). Ranges that may start or end inside a packet (`base_aligned`
// false, or a range length that is not whole packets) keep two packets for
// their ends.
inline bool plan_short_rows(int64_t C, size_t elem_bytes, int packets_per_thread,
                            bool base_aligned, ShortPlan* p) {
  if (C > 1024) return false;
  int lanes = 4;
  while (lanes < 64 && C > lanes * 8) lanes <<= 1;
  p->lanes = lanes;
  p->per_lane = C <= lanes * 8 ? 8 : 16;
  const size_t row_bytes = static_cast<size_t>(C) * elem_bytes;
  const uint32_t per_pass = kShortThreads / lanes;
  const size_t slots = static_cast<size_t>(kShortThreads) * packets_per_thread;
  auto rows_for = [&](size_t capacity) {
    uint32_t rows = static_cast<uint32_t>(capacity / row_bytes);
    rows = rows / per_pass * per_pass;
    if (rows > slots) rows = static_cast<uint32_t>(slots / per_pass * per_pass);  // one scalar slot per row
    return rows;
  };
  uint32_t rows = rows_for(slots * 16);
  if (rows == 0 || !base_aligned || (rows * row_bytes) % 16 != 0) rows = rows_for((slots - 2) * 16);
  if (rows == 0) rows = per_pass;  // at least one row per lane group (at most 16 KB)
  p->rows_per_chunk = rows;
  p->stage_packets = static_cast<uint32_t>((rows * row_bytes + 15) / 16 + 2);
  return true;
}
// The plan with the most packets per thread, up to `packets_per_thread`, whose
// LDS need `lds_of(plan)` (stage plus per-row scalars) stays within the 48 KB a
// kernel may use without its limit being raised.
template <typename LdsOf>
inline bool plan_short_rows_within(int64_t C, size_t elem_bytes, int packets_per_thread,
                                   bool base_aligned, LdsOf lds_of, ShortPlan* p) {
  for (int ppt = packets_per_thread; ppt >= 1; --ppt) {
    if (!plan_short_rows(C, elem_bytes, ppt, base_aligned, p)) return false;
    if (lds_of(*p) <= 48 * 1024) return true;
  }
  return false;  // even one packet per thread needs more: the caller takes its next path
}
inline unsigned short_grid(int64_t N, uint32_t rows_per_chunk) {
  const int64_t chunks = ceil_div(N, rows_per_chunk);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 16;
  return static_cast<unsigned>(chunks < cap ? chunks : cap);
}

// Launches short_rows<T, L, E, OP<T, E>> for the plan; OP is the policy
// template, the trailing arguments its constructor arguments.
#define DRAGON_HIP_SHORT_LAUNCH(T, OP, sp, lds, grid, stream, N, C, in0, in1, out, ...)        \
  {                                                                                          \
    const dim3 g_(grid), b_(kShortThreads);                                                  \
    if (sp.per_lane == 8) {                                                                  \
      const OP<T, 8> op_{__VA_ARGS__};                                                       \
      if (sp.lanes == 4)                                                                     \
        hipLaunchKernelGGL((short_rows<T, 4, 8, OP<T, 8>>), g_, b_, lds, stream, N, C,   \
                           sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);         \
      else if (sp.lanes == 8)                                                                \
        hipLaunchKernelGGL((short_rows<T, 8, 8, OP<T, 8>>), g_, b_, lds, stream, N, C,   \
                           sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);         \
      else if (sp.lanes == 16)                                                               \
        hipLaunchKernelGGL((short_rows<T, 16, 8, OP<T, 8>>), g_, b_, lds, stream, N, C,  \
                           sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);         \
      else if (sp.lanes == 32)                                                               \
        hipLaunchKernelGGL((short_rows<T, 32, 8, OP<T, 8>>), g_, b_, lds, stream, N, C,  \
                           sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);         \
      else                                                                                   \
        hipLaunchKernelGGL((short_rows<T, 64, 8, OP<T, 8>>), g_, b_, lds, stream, N, C,  \
                           sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);         \
    } else {                                                                                 \
      const OP<T, 16> op_{__VA_ARGS__};                                                      \
      hipLaunchKernelGGL((short_rows<T, 64, 16, OP<T, 16>>), g_, b_, lds, stream, N, C,  \
                         sp.rows_per_chunk, sp.stage_packets, in0, in1, out, op_);           \
    }                                                                                        \
  }

} // namespace dragon_hip
