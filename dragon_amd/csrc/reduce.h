// Atomic-free two-stage reductions and flat element-wise maps shared by the
// Moments, GroupNorm and BatchNorm kernels.
//
// Every reduction on this path is a pair of sums per output (sum x / sum x^2,
// sum dy*(x-mu) / sum dy, sum gamma*dy*x / sum gamma*dy ...). Stage one spreads
// each output over `split` workgroups so that a few hundred outputs still fill
// 256 compute units; each workgroup tree-reduces its share in fp32 (fp64 for
// double) and writes one pair to scratch. Stage two is a tiny kernel that adds
// the `split` pairs of an output in a fixed order and applies the op's
// epilogue. No atomics, so results are bit-reproducible run to run.
//
// Sizes: the reference's kernels:: interface carries `int` extents
// (dragon/kernels/normalization/op_kernels.h:36-143), so every tensor on this
// path has fewer than 2^31 elements and 32-bit index arithmetic is exact.
#pragma once

#include "common.h"

namespace dragon_hip {

constexpr int kReduceThreads = 256;
constexpr int kReduceWaves = kReduceThreads / kWaveSize;

// Reduction set of output o = (o1, o2), o = o1 * outer2 + o2: `nseg` segments
// of `seglen` contiguous elements; element (seg, p) lives at
//   o1 * stride1 + o2 * stride2 + seg * seg_stride + p.
//   trailing-axis reduce [rows, cols]   outer2=1, stride1=cols, nseg=1, seglen=cols
//   BatchNorm NCHW [N, C, S] per c      outer2=C, stride2=S, nseg=N, seg_stride=C*S, seglen=S
//   GroupNorm NCHW per (n, g)           outer2=1, stride1=D*S, nseg=1, seglen=D*S
//   GroupNorm NHWC per (n, g)           outer2=G, stride1=S*C, stride2=D, nseg=S, seg_stride=C, seglen=D
struct SegmentedReduce {
  uint32_t n_out, outer2;
  uint32_t stride1, stride2;
  uint32_t nseg, seglen, seg_stride;
  uint32_t split;
};

// Leading-axis reduce of a [rows, cols] view, one output per column
// (BatchNorm NHWC, parameter gradients of row-normalised tensors).
struct ColumnReduce {
  uint32_t rows, cols;
  uint32_t split;
};

// How many workgroups share one output: enough to put ~8 workgroups on every
// compute unit, but never less than ~16K elements per workgroup. Rounded down:
// a few workgroups more than the device holds at once would run as a second,
// nearly empty round (48 column tiles x 43 = 2064 workgroups on 256 compute
// units: 88 us; x 42: one round).
inline uint32_t pick_split(int64_t n_out, int64_t elems_per_out) {
  const int64_t want_blocks = static_cast<int64_t>(num_cus()) * 8;
  int64_t split = want_blocks / (n_out > 0 ? n_out : 1);
  const int64_t max_by_work = ceil_div(elems_per_out, 16384);
  if (split > max_by_work) split = max_by_work;
  if (split < 1) split = 1;
  if (split > 1024) split = 1024;
  return static_cast<uint32_t>(split);
}

template <typename A>
__device__ __forceinline__ void block_reduce_pair(A& a, A& b, A* lds /*2*kReduceWaves*/) {
  a = wave_allreduce(a, SumOp());
  b = wave_allreduce(b, SumOp());
  const int wave = threadIdx.x / kWaveSize;
  if ((threadIdx.x & (kWaveSize - 1)) == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  __syncthreads();
  a = lds[0], b = lds[1];
#pragma unroll
  for (int i = 1; i < kReduceWaves; ++i) {
    a += lds[2 * i];
    b += lds[2 * i + 1];
  }
}

// Stage one over segments. F provides
//   void begin(uint32_t o, uint32_t first_off)    per-output setup; first_off is
//                                                 the offset of the output's first element
//   void add(uint32_t o, uint32_t seg, uint32_t p, uint32_t off,
//            const A (&x0)[V], const A (&x1)[V], A& a, A& b)
// where `off` is the element offset of the packet; kVec == 1 is the scalar
// variant for unaligned tensors. partial[(o * split + k) * 2 + {0,1}].
template <typename T, int kIn, int kVec, typename F>
__global__ __launch_bounds__(kReduceThreads) void reduce2_segments(
    const SegmentedReduce d, const T* __restrict__ in0, const T* __restrict__ in1, F f,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds[2 * kReduceWaves];
  const uint32_t o = blockIdx.x / d.split;
  const uint32_t k = blockIdx.x - o * d.split;
  const uint32_t o1 = o / d.outer2;
  const uint32_t o2 = o - o1 * d.outer2;
  const uint32_t base = o1 * d.stride1 + o2 * d.stride2;
  const uint32_t packets_per_seg = d.seglen / kVec;  // kVec > 1 only when it divides seglen
  const uint32_t npackets = d.nseg * packets_per_seg;
  f.begin(o, base);
  A a = A(0), b = A(0);
#pragma unroll 4
  for (uint32_t jp = k * kReduceThreads + threadIdx.x; jp < npackets;
       jp += d.split * kReduceThreads) {
    const uint32_t seg = jp / packets_per_seg;
    const uint32_t p = (jp - seg * packets_per_seg) * kVec;
    const uint32_t off = base + seg * d.seg_stride + p;
    A x0[kVec], x1[kVec];
    if constexpr (kVec == 1) {
      x0[0] = IO<T>::load1(in0 + off);
      x1[0] = kIn == 2 ? IO<T>::load1(in1 + off) : A(0);
    } else {
      load_unpack_keep<T>(in0 + off, x0);
      if constexpr (kIn == 2) load_unpack_keep<T>(in1 + off, x1);
    }
    f.add(o, seg, p, off, x0, x1, a, b);
  }
  block_reduce_pair(a, b, lds);
  if (threadIdx.x == 0) {
    partial[(static_cast<size_t>(o) * d.split + k) * 2] = a;
    partial[(static_cast<size_t>(o) * d.split + k) * 2 + 1] = b;
  }
}

// Stage one over segments of any length at any element-aligned address, read as
// the aligned 16-byte packets that cover each segment (two tensors must be
// congruent modulo 16 bytes): a segment of seglen elements takes
// seglen / kVec + 2 packet slots, of which the last may lie wholly behind it
// and is skipped. A packet wholly inside its segment goes to F's packet
// interface; the elements of a segment in its first and last packet go to the
// scalar one, one call per element, so F sees exactly the elements and indices
// it would see element by element. An aligned packet that holds a byte of a
// tensor lies in that byte's page, so packets that reach beyond a tensor's ends
// may be read whole.
template <typename T, int kIn, typename F>
__global__ __launch_bounds__(kReduceThreads) void reduce2_segments_windows(
    const SegmentedReduce d, const T* __restrict__ in0, const T* __restrict__ in1, F f,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  __shared__ A lds[2 * kReduceWaves];
  const uint32_t o = blockIdx.x / d.split;
  const uint32_t k = blockIdx.x - o * d.split;
  const uint32_t o1 = o / d.outer2;
  const uint32_t o2 = o - o1 * d.outer2;
  const uint32_t base = o1 * d.stride1 + o2 * d.stride2;
  const uint32_t slots_per_seg = d.seglen / kVec + 2;
  const uint32_t nslots = d.nseg * slots_per_seg;
  f.begin(o, base);
  A a = A(0), b = A(0);
#pragma unroll 4
  for (uint32_t js = k * kReduceThreads + threadIdx.x; js < nslots;
       js += d.split * kReduceThreads) {
    const uint32_t seg = js / slots_per_seg;
    const uint32_t q = js - seg * slots_per_seg;
    const uint32_t s0 = base + seg * d.seg_stride;  // the segment's first element
    const int lead = static_cast<int>((reinterpret_cast<uintptr_t>(in0 + s0) & 15u) / sizeof(T));
    const int pe = static_cast<int>(q * kVec) - lead;  // the packet's first element, in the segment
    if (pe >= static_cast<int>(d.seglen)) continue;
    A x0[kVec], x1[kVec];
    load_unpack_keep<T>(in0 + (static_cast<int64_t>(s0) + pe), x0);
    if constexpr (kIn == 2) load_unpack_keep<T>(in1 + (static_cast<int64_t>(s0) + pe), x1);
    if (pe >= 0 && pe + kVec <= static_cast<int>(d.seglen)) {
      f.add(o, seg, static_cast<uint32_t>(pe), s0 + pe, x0, x1, a, b);
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (pe + e >= 0 && pe + e < static_cast<int>(d.seglen)) {
          const A y0[1] = {x0[e]};
          const A y1[1] = {kIn == 2 ? x1[e] : A(0)};
          f.add(o, seg, static_cast<uint32_t>(pe + e), s0 + pe + e, y0, y1, a, b);
        }
      }
    }
  }
  block_reduce_pair(a, b, lds);
  if (threadIdx.x == 0) {
    partial[(static_cast<size_t>(o) * d.split + k) * 2] = a;
    partial[(static_cast<size_t>(o) * d.split + k) * 2 + 1] = b;
  }
}

// Stage one over columns: a workgroup owns a tile of 64 adjacent columns
// (one per lane, so a wavefront reads 64 adjacent elements) and its four
// wavefronts stride over the rows of slice k. F provides
//   void begin(uint32_t c, uint32_t first_off)
//   void add(uint32_t r, uint32_t c, uint32_t off, A x0, A x1, A& a, A& b).
// partial[(k * cols + c) * 2 + {0,1}].
template <typename T, int kIn, typename F>
__global__ __launch_bounds__(kReduceThreads) void reduce2_columns(
    const ColumnReduce d, const uint32_t lanes_per_row, const T* __restrict__ in0,
    const T* __restrict__ in1, F f, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds[kReduceWaves][kWaveSize][2];
  // fewer than 64 columns: the lanes a row does not need take adjacent rows
  // (as reduce2_columns_packets below)
  const uint32_t rows_per_wave = kWaveSize / lanes_per_row;
  const uint32_t tiles = (d.cols + lanes_per_row - 1) / lanes_per_row;
  const uint32_t tile = blockIdx.x % tiles;
  const uint32_t k = blockIdx.x / tiles;
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t across = lane / lanes_per_row;
  const uint32_t c = tile * lanes_per_row + lane % lanes_per_row;
  A a = A(0), b = A(0);
  if (c < d.cols) {
    f.begin(c, c);
#pragma unroll 4
    for (uint32_t r = (k * kReduceWaves + wave) * rows_per_wave + across; r < d.rows;
         r += d.split * kReduceWaves * rows_per_wave) {
      const uint32_t off = r * d.cols + c;
      const A x0 = IO<T>::load1(in0 + off);
      const A x1 = kIn == 2 ? IO<T>::load1(in1 + off) : A(0);
      f.add(r, c, off, x0, x1, a, b);
    }
  }
  for (uint32_t o = lanes_per_row; o < kWaveSize; o <<= 1) {
    a += __shfl_xor(a, static_cast<int>(o), kWaveSize);
    b += __shfl_xor(b, static_cast<int>(o), kWaveSize);
  }
  lds[wave][lane][0] = a;
  lds[wave][lane][1] = b;
  __syncthreads();
  if (wave == 0 && across == 0 && c < d.cols) {
#pragma unroll
    for (int w = 1; w < kReduceWaves; ++w) {
      a += lds[w][lane][0];
      b += lds[w][lane][1];
    }
    partial[(static_cast<size_t>(k) * d.cols + c) * 2] = a;
    partial[(static_cast<size_t>(k) * d.cols + c) * 2 + 1] = b;
  }
}

// The same with a 16-byte packet of kVec adjacent columns per lane (cols a
// multiple of kVec, 16-byte aligned base): a wavefront reads 1 KiB at a time.
// `lanes_per_row` lanes lie along a row: the whole wavefront, or, for a matrix
// of fewer than 64 packets per row, the power of two that covers a row, the
// remaining lane bits taking adjacent rows (so that 32 sixteen-bit channels do
// not leave 60 of 64 lanes idle). Each column keeps its own copy of the
// accumulator functor.
template <typename T, int kIn, typename F>
__global__ __launch_bounds__(kReduceThreads) void reduce2_columns_packets(
    const ColumnReduce d, const uint32_t lanes_per_row, const T* __restrict__ in0,
    const T* __restrict__ in1, F f, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  __shared__ A lds[kReduceWaves][kWaveSize][2 * kVec];
  const uint32_t rows_per_wave = kWaveSize / lanes_per_row;
  const uint32_t tile_cols = lanes_per_row * kVec;
  const uint32_t tiles = (d.cols + tile_cols - 1) / tile_cols;
  const uint32_t tile = blockIdx.x % tiles;
  const uint32_t k = blockIdx.x / tiles;
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t along = lane % lanes_per_row, across = lane / lanes_per_row;
  const uint32_t c0 = tile * tile_cols + along * kVec;
  A a[kVec], b[kVec];
#pragma unroll
  for (int e = 0; e < kVec; ++e) a[e] = b[e] = A(0);
  if (c0 < d.cols) {
    F fs[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      fs[e] = f;
      fs[e].begin(c0 + e, c0 + e);
    }
#pragma unroll 4
    for (uint32_t r = (k * kReduceWaves + wave) * rows_per_wave + across; r < d.rows;
         r += d.split * kReduceWaves * rows_per_wave) {
      const uint32_t off = r * d.cols + c0;
      A x0[kVec], x1[kVec];
      load_unpack_keep<T>(in0 + off, x0);
      if constexpr (kIn == 2) load_unpack_keep<T>(in1 + off, x1);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        fs[e].add(r, c0 + e, off + e, x0[e], kIn == 2 ? x1[e] : A(0), a[e], b[e]);
      }
    }
  }
  // the lanes that share a column (uniform trip count: every lane takes part)
  for (uint32_t o = lanes_per_row; o < kWaveSize; o <<= 1) {
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      a[e] += __shfl_xor(a[e], static_cast<int>(o), kWaveSize);
      b[e] += __shfl_xor(b[e], static_cast<int>(o), kWaveSize);
    }
  }
#pragma unroll
  for (int e = 0; e < kVec; ++e) {
    lds[wave][lane][2 * e] = a[e];
    lds[wave][lane][2 * e + 1] = b[e];
  }
  __syncthreads();
  if (wave == 0 && across == 0 && c0 < d.cols) {
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
#pragma unroll
      for (int w = 1; w < kReduceWaves; ++w) {
        a[e] += lds[w][lane][2 * e];
        b[e] += lds[w][lane][2 * e + 1];
      }
      partial[(static_cast<size_t>(k) * d.cols + c0 + e) * 2] = a[e];
      partial[(static_cast<size_t>(k) * d.cols + c0 + e) * 2 + 1] = b[e];
    }
  }
}

// The largest split any column stage one chooses for a [rows, cols] reduction
// (the packet kernel, with the fewest tiles, splits the rows finest): sizes the
// scratch, split * cols pairs.
inline uint32_t column_split_bound(int64_t rows, int64_t cols) {
  return pick_split(ceil_div(cols, kWaveSize * 8), rows * kWaveSize * 8);
}
// Launches the column stage one that suits the shape and returns its split.
template <typename T, int kIn, typename F>
inline uint32_t launch_reduce2_columns(uint32_t rows, uint32_t cols, const T* in0, const T* in1,
                                       F f, typename IO<T>::Acc* partial, hipStream_t stream) {
  constexpr int kVec = IO<T>::kVec;
  ColumnReduce d{rows, cols, 1};
  const bool packets = cols % kVec == 0 && aligned16(in0) && (kIn == 1 || aligned16(in1));
  if (packets) {
    uint32_t lanes_per_row = 1;
    while (lanes_per_row < kWaveSize && lanes_per_row * kVec < cols) lanes_per_row <<= 1;
    uint32_t tiles = static_cast<uint32_t>(ceil_div(cols, lanes_per_row * kVec));
    // A row of 40, 48 or 80 packets (320, 384, 640 sixteen-bit channels) leaves a
    // quarter or more of the 64-lane tiles idle: tiles of the largest power of two
    // that divides the row (128 bytes or more of a row per tile) keep every lane busy.
    const uint32_t row_packets = cols / kVec;
    if (static_cast<uint64_t>(row_packets) * 5 < static_cast<uint64_t>(tiles) * lanes_per_row * 4) {
      const uint32_t pow2 = row_packets & (~row_packets + 1);  // largest power of two dividing it
      if (pow2 >= 8 && pow2 < lanes_per_row) {
        lanes_per_row = pow2;
        tiles = row_packets / pow2;
      }
    }
    d.split = pick_split(tiles, static_cast<int64_t>(rows) * kWaveSize * kVec);
    // The pairs are written once and read once, 16 bytes per column and split
    // against rows * sizeof(T) bytes of input per column: where that is more
    // than a twelfth, half as many workgroups with twice the rows each.
    if (static_cast<int64_t>(d.split) * 16 * 12 > static_cast<int64_t>(rows) * sizeof(T)) {
      d.split = (d.split + 1) / 2;
    }
    hipLaunchKernelGGL((reduce2_columns_packets<T, kIn, F>), dim3(tiles * d.split),
                       dim3(kReduceThreads), 0, stream, d, lanes_per_row, in0, in1, f, partial);
  } else {
    uint32_t lanes_per_row = 1;
    while (lanes_per_row < kWaveSize && lanes_per_row < cols) lanes_per_row <<= 1;
    const uint32_t tiles = static_cast<uint32_t>(ceil_div(cols, lanes_per_row));
    d.split = pick_split(tiles, static_cast<int64_t>(rows) * kWaveSize);
    hipLaunchKernelGGL((reduce2_columns<T, kIn, F>), dim3(tiles * d.split), dim3(kReduceThreads), 0,
                       stream, d, lanes_per_row, in0, in1, f, partial);
  }
  return d.split;
}

// Stage two: one thread per output adds its `split` pairs in index order and
// hands the totals to the epilogue E: void operator()(uint32_t o, A a, A b).
// `segment_major` selects the scratch layout of reduce2_segments
// ((o*split+k)*2) or of reduce2_columns ((k*n_out+o)*2).
template <typename A, typename E>
__global__ __launch_bounds__(kReduceThreads) void reduce2_finalize(
    const uint32_t n_out, const uint32_t split, const bool segment_major,
    const A* __restrict__ partial, E e) {
  const uint32_t o = blockIdx.x * kReduceThreads + threadIdx.x;
  if (o >= n_out) return;
  A a = A(0), b = A(0);
  for (uint32_t k = 0; k < split; ++k) {
    const size_t idx = segment_major ? (static_cast<size_t>(o) * split + k)
                                     : (static_cast<size_t>(k) * n_out + o);
    a += partial[idx * 2];
    b += partial[idx * 2 + 1];
  }
  e(o, a, b);
}

// Stage two for the scratch layout of reduce2_columns when `split` is large:
// a 1024-thread workgroup owns 16 adjacent outputs; thread (ol, kl) sums the
// pairs k = kl, kl + 64, ... of output ol (a wavefront reads four runs of 16
// adjacent pairs), the four k-lanes of a wavefront are combined by shuffles
// and the sixteen wavefronts in wavefront order through LDS. Fixed summation
// order, like reduce2_finalize.
constexpr int kFinalizeThreads = 1024;
constexpr int kFinalizeOutputs = 16;
constexpr int kFinalizeWaves = kFinalizeThreads / kWaveSize;
template <typename A, typename E>
__global__ __launch_bounds__(kFinalizeThreads) void reduce2_finalize_columns(
    const uint32_t n_out, const uint32_t split, const A* __restrict__ partial, E e) {
  __shared__ A lds[kFinalizeWaves][kFinalizeOutputs][2];
  const uint32_t ol = threadIdx.x & (kFinalizeOutputs - 1);
  const uint32_t kl = threadIdx.x / kFinalizeOutputs;
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t o = blockIdx.x * kFinalizeOutputs + ol;
  A a = A(0), b = A(0);
  if (o < n_out) {
#pragma unroll 8
    for (uint32_t k = kl; k < split; k += kFinalizeThreads / kFinalizeOutputs) {
      const size_t idx = static_cast<size_t>(k) * n_out + o;
      a += partial[idx * 2];
      b += partial[idx * 2 + 1];
    }
  }
#pragma unroll
  for (int off = kFinalizeOutputs; off < kWaveSize; off <<= 1) {
    a += __shfl_xor(a, off, kWaveSize);
    b += __shfl_xor(b, off, kWaveSize);
  }
  if ((threadIdx.x & (kWaveSize - 1)) < kFinalizeOutputs) {
    lds[wave][ol][0] = a;
    lds[wave][ol][1] = b;
  }
  __syncthreads();
  if (threadIdx.x < kFinalizeOutputs && o < n_out) {
    a = lds[0][ol][0], b = lds[0][ol][1];
#pragma unroll
    for (int w = 1; w < kFinalizeWaves; ++w) {
      a += lds[w][ol][0];
      b += lds[w][ol][1];
    }
    e(o, a, b);
  }
}

// Launches the stage-two kernel that suits the layout and the split.
template <typename A, typename E>
inline void launch_reduce2_finalize(uint32_t n_out, uint32_t split, bool segment_major,
                                    const A* partial, E e, hipStream_t stream) {
  if (!segment_major && split > 16) {
    hipLaunchKernelGGL((reduce2_finalize_columns<A, E>),
                       dim3((n_out + kFinalizeOutputs - 1) / kFinalizeOutputs),
                       dim3(kFinalizeThreads), 0, stream, n_out, split, partial, e);
  } else {
    hipLaunchKernelGGL((reduce2_finalize<A, E>), dim3((n_out + kReduceThreads - 1) / kReduceThreads),
                       dim3(kReduceThreads), 0, stream, n_out, split, segment_major, partial, e);
  }
}

// Flat element-wise map over `total` elements in packets of kVec. F provides
//   void operator()(uint32_t i, A (&v0)[V], const A (&v1)[V])
// which overwrites v0 (loaded from in0) with the result; v1 comes from in1
// when kIn == 2.
template <typename T, int kIn, int kVec, typename F>
__global__ __launch_bounds__(256) void map_flat(const uint32_t total, const T* in0, const T* in1,
                                                T* out, F f) {
  using A = typename IO<T>::Acc;
  const uint32_t npackets = total / kVec;  // kVec > 1 only when it divides total
  for (uint32_t ip = blockIdx.x * 256 + threadIdx.x; ip < npackets; ip += gridDim.x * 256) {
    const uint32_t i = ip * kVec;
    A v0[kVec], v1[kVec];
    if constexpr (kVec == 1) {
      v0[0] = IO<T>::load1(in0 + i);
      v1[0] = kIn == 2 ? IO<T>::load1(in1 + i) : A(0);
    } else {
      load_unpack<T>(in0 + i, v0);
      if constexpr (kIn == 2) load_unpack<T>(in1 + i, v1);
    }
    f(i, v0, v1);
    if constexpr (kVec == 1) {
      IO<T>::store1(out + i, v0[0]);
    } else {
      pack_store<T>(out + i, v0);
    }
  }
}

// An element-wise map with per-run parameters over a tensor whose runs of
// `run` elements (the feature maps of an NCHW tensor) are not whole packets, or
// that starts at an element-aligned address (all tensors congruent modulo 16
// bytes): the aligned 16-byte packets that cover the tensor. Op provides
//   static constexpr int kParams;  void row_params(int64_t r, A (&w)[kParams]) const
//   A apply(const A* w, A x0, A x1) const
// (the interface of long_rows_map). The run is found once per packet; a packet
// that straddles two runs takes the next run's parameters from the boundary on. Of the packets that reach beyond the tensor's ends only the
// tensor's own elements are computed and stored. An aligned packet that holds
// a byte of the tensor lies in that byte's page, so those may be read whole.
template <typename T, int kIn, typename Op>
__global__ __launch_bounds__(256) void map_flat_windows(const uint32_t total, const uint32_t run,
                                                        const T* in0, const T* in1, T* out,
                                                        const Op f) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const int lead = static_cast<int>((reinterpret_cast<uintptr_t>(in0) & 15u) / sizeof(T));
  const uint32_t npackets = (static_cast<uint32_t>(lead) + total + kVec - 1) / kVec;
  for (uint32_t ip = blockIdx.x * 256 + threadIdx.x; ip < npackets; ip += gridDim.x * 256) {
    const int64_t i = static_cast<int64_t>(ip) * kVec - lead;  // the packet's first element
    A v0[kVec], v1[kVec];
    load_unpack<T>(in0 + i, v0);
    if constexpr (kIn == 2) load_unpack<T>(in1 + i, v1);
    const bool inside = i >= 0 && i + kVec <= static_cast<int64_t>(total);
    const uint32_t first = static_cast<uint32_t>(i < 0 ? 0 : i);  // first element inside the tensor
    const uint32_t r = first / run;
    // elements of the packet, counted from `first`, that still lie in run r
    const uint32_t left = (r + 1) * run - first;
    A w[Op::kParams];
    f.row_params(r, w);
    if (inside && left >= static_cast<uint32_t>(kVec)) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) v0[e] = f.apply(w, v0[e], kIn == 2 ? v1[e] : A(0));
      pack_store<T>(out + i, v0);
    } else {
      A w2[Op::kParams];
      f.row_params((r + 2) * run <= total ? r + 1 : r, w2);  // (no run behind the last one)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const int64_t j = i + e;
        if (j >= 0 && j < static_cast<int64_t>(total)) {
          const bool next = static_cast<uint32_t>(j) - first >= left;
          v0[e] = f.apply(next ? w2 : w, v0[e], kIn == 2 ? v1[e] : A(0));
          if (!inside) IO<T>::store1(out + j, v0[e]);
        }
      }
      if (inside) pack_store<T>(out + i, v0);
    }
  }
}

inline unsigned map_grid(uint32_t npackets) {
  const int64_t want = ceil_div(npackets, 256);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 32;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

inline bool fits_int32(int64_t v) { return v >= 0 && v < (int64_t(1) << 31); }

} // namespace dragon_hip
