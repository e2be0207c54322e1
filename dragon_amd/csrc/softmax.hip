// Softmax / LogSoftmax forward and backward for gfx950.
//
// Replaces kernels::Softmax, LogSoftmax, SoftmaxGrad, LogSoftmaxGrad
// (dragon/kernels/activation/op_kernels.h:211-247; CPU
// dragon/kernels/activation/cpu/softmax_kernel.cc:10-108) over a tensor viewed
// as [N, C, S] with the reduction along C:
//   softmax       y  = exp(x - max) / sum exp(x - max)
//   log_softmax   y  = (x - max) - log sum exp(x - max)
//   softmax_grad      dx = (dy - sum(dy * y)) * y
//   log_softmax_grad  dx = dy - exp(y) * sum(dy)
//
// S == 1 (reduction along the contiguous axis) keeps each row in registers:
// every tensor is read once and written once, whatever the row width and
// alignment (ragged tiles take widths that are not whole 16-byte packets). 16-bit I/O accumulates in fp32
// and uses the hardware exp2 (relative error ~1e-7 near the row maximum,
// below 3e-6 in the far tail, both far under one 16-bit ulp); fp32 / fp64 I/O
// use the library exp. fp32 multiplies by the reciprocal of the row sum (one
// ulp from the reference's quotient), fp64 divides as the reference does.
//
// S > 1 keeps a [C, columns] tile in the registers of a workgroup (col_tile.h)
// when C <= 1024: one read, one write. Longer strided
// axes assign one thread to each (n, s) column and walk it three times (max,
// sum, write), the re-reads coming from L2.
#include "col_tile.h"
#include "loss_math.h"
#include "row_loop.h"
#include "row_tile.h"
#include "short_rows.h"
#include "slices.h"

namespace dragon_hip {
namespace {

template <typename T>
struct SoftmaxMath {
  using A = typename IO<T>::Acc;
  static constexpr bool kFast = sizeof(T) == 2;
  static __device__ __forceinline__ A exp_of(A v) {
    if constexpr (kFast) {
      return __builtin_amdgcn_exp2f(v * 1.44269504088896340736f);
    } else {
      return acc_exp(v);
    }
  }
  // fp32 and 16-bit outputs multiply by the correctly rounded reciprocal of the
  // sum (within one fp32 ulp of the quotient, a tenth of a microsecond-scale
  // division sequence per element saved); fp64 divides.
  static __device__ __forceinline__ A normalise(A e, A sum, A inv_sum) {
    if constexpr (sizeof(A) == 4) {
      return e * inv_sum;
    } else {
      return e / sum;
    }
  }
};

enum SoftmaxKind { kSoftmax = 0, kLogSoftmax = 1 };

// Rows held in registers by kTPR threads; a wavefront that holds a whole row in
// one or two packets per lane takes two neighbouring rows at a time
// (wave_rows_at_a_time).
template <typename T, int kKind, int kTPR, int kVPT, bool kRagged, bool kFull = false,
          bool kWindow = false>
__global__ __launch_bounds__(row_threads(kTPR)) void softmax_rows(
    const int64_t N, const int C, const T* x, T* y) {
  static_assert(!(kWindow && (kRagged || kFull)), "windows use the regular tile");
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  constexpr int kR = wave_rows_at_a_time<kTPR, kVPT>();
  constexpr int kRowsPerStep = Tile::kRowsPerBlock * kR;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = Tile::extent_of(C);

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerStep + Tile::sub_row() * kR;
       row < N; row += static_cast<int64_t>(gridDim.x) * kRowsPerStep) {
    Tile t[kR];
    bool on[kR];  // uniform over the row's threads
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      on[r] = row + r < N;
      const T* src = x + (on[r] ? row + r : row) * C;
      if constexpr (kWindow) {
        t[r].load_window(src, RowWindow<T>(src, C), acc_neg_inf<A>());
      } else if constexpr (kFull) {
        t[r].load_full(src);  // the row fills the tile: nothing to mask
      } else {
        t[r].load(src, npackets, acc_neg_inf<A>());
      }
    }

    A m[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      m[r] = acc_neg_inf<A>();
#pragma unroll
      for (int i = 0; i < kVPT; ++i)
#pragma unroll
        for (int e = 0; e < kVec; ++e) m[r] = MaxOp()(m[r], t[r].v[i][e]);
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) m[r] = Tile::reduce(m[r], MaxOp(), slots[0]);

    A s[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      s[r] = A(0);
#pragma unroll
      for (int i = 0; i < kVPT; ++i)
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (kKind == kSoftmax) {
            t[r].v[i][e] = M::exp_of(t[r].v[i][e] - m[r]);  // masked slots: exp(-inf) = 0
            s[r] += t[r].v[i][e];
          } else {
            t[r].v[i][e] = t[r].v[i][e] - m[r];
            s[r] += M::exp_of(t[r].v[i][e]);
          }
        }
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) s[r] = Tile::reduce(s[r], SumOp(), slots[1]);

#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (kKind == kSoftmax) {
        const A inv = A(1) / s[r];
#pragma unroll
        for (int i = 0; i < kVPT; ++i)
#pragma unroll
          for (int e = 0; e < kVec; ++e) t[r].v[i][e] = M::normalise(t[r].v[i][e], s[r], inv);
      } else {
        const A l = acc_log(s[r]);
#pragma unroll
        for (int i = 0; i < kVPT; ++i)
#pragma unroll
          for (int e = 0; e < kVec; ++e) t[r].v[i][e] = t[r].v[i][e] - l;
      }
      if constexpr (kWindow) {
        if (on[r]) t[r].store_window(y + (row + r) * C, RowWindow<T>(x + (row + r) * C, C));
      } else {
        if (on[r]) t[r].store(y + (row + r) * C, npackets);
      }
    }
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// Rows that take a whole 1024-thread workgroup (a compute unit holds one or
// two of those): a persistent workgroup requests the next row's packets before
// it reduces the current row, and issues the current row's stores after the
// wait for them, so loads, arithmetic and stores of neighbouring rows overlap.
// The ragged flavour takes rows of any width at element-aligned addresses and
// reads whole packets, up to kVec - 1 elements past a row's end: the caller
// gives it all rows but the tensor's last.
template <typename T, int kKind, int kVPT, bool kRagged = false>
__global__ __launch_bounds__(1024) void softmax_wide_rows(const int64_t N, const int C, const T* x,
                                                          T* y) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT, kTPR, kRagged>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = Tile::extent_of(C);  // columns for the ragged flavour
  // the row's last packet when it is partial: its slot, lane and element count
  const int tail_valid = C % kVec;
  const int tail_slot = tail_valid ? (C / kVec) / kTPR : -1;
  const int tail_lane = (C / kVec) % kTPR;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  Raw cur;
  if constexpr (kRagged) {
    cur.load_over(x + (row < N ? row : 0) * C, C, row < N);
  } else {
    cur.load(x + (row < N ? row : 0) * C, npackets, row < N);
  }
  for (; row < N; row += stride) {
    Raw nxt;
    const bool more = row + stride < N;
    if constexpr (kRagged) {
      nxt.load_over(x + (more ? row + stride : 0) * C, C, more);
    } else {
      nxt.load(x + (more ? row + stride : 0) * C, npackets, more);
    }
    Tile t;
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      cur.unpack(i, t.v[i]);
      const bool on = Tile::active(i, npackets);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = on ? t.v[i][e] : acc_neg_inf<A>();  // raw padding is zero bits
      }
      if constexpr (kRagged) {
        // only the slot of the row's last, partial packet holds elements past the row
        if (i == tail_slot) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (Tile::lane() == tail_lane && e >= tail_valid) t.v[i][e] = acc_neg_inf<A>();
          }
        }
      }
#pragma unroll
      for (int e = 0; e < kVec; ++e) m = MaxOp()(m, t.v[i][e]);
    }
    m = Tile::reduce(m, MaxOp(), slots[0]);
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (kKind == kSoftmax) {
          t.v[i][e] = M::exp_of(t.v[i][e] - m);
          s += t.v[i][e];
        } else {
          t.v[i][e] = t.v[i][e] - m;
          s += M::exp_of(t.v[i][e]);
        }
      }
    s = Tile::reduce(s, SumOp(), slots[1]);
    const A inv = A(1) / s;
    const A l = acc_log(s);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = kKind == kSoftmax ? M::normalise(t.v[i][e], s, inv) : t.v[i][e] - l;
      }
    nxt.wait_ready();
    cur = nxt;
    if constexpr (kRagged) {
      T* out = y + row * C;
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        const int col = (i * kTPR + Tile::lane()) * kVec;
        if (i == tail_slot && Tile::lane() == tail_lane) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (e < tail_valid) IO<T>::store1(out + col + e, t.v[i][e]);
          }
        } else if (col < C) {
          store_packet_unaligned(out + col, IO<T>::pack(t.v[i]));
        }
      }
    } else {
      t.store(y + row * C, npackets);
    }
    __syncthreads();  // slots are reused by the next row
  }
}

// softmax_wide_rows for rows that are not whole aligned packets, through their
// windows; x and y must be congruent modulo 16 bytes. A window may be one packet
// longer than the row has whole packets: the caller picks kVPT for C / kVec + 2
// packets. What the window's first and last packet hold of the neighbouring rows
// is set to -inf in the two lanes concerned before the row is reduced, so the
// passes are those of rows of whole packets; those two packets go through LDS
// and are stored element by element by the first threads of the workgroup.
template <typename T, int kKind, int kVPT>
__global__ __launch_bounds__(1024) void softmax_wide_windows(const int64_t N, const int C,
                                                             const T* x, T* y) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT, kTPR, false>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  __shared__ u32x4 edge[2];
  const int lane = threadIdx.x;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  auto request = [&](Raw& t, const int64_t at, const bool valid) {
    const int64_t from = valid ? at : 0;
    const RowWindow<T> w(x + from * C, C);
    t.load(x + from * C - w.lead, w.packets, valid);
  };
  Raw cur;
  request(cur, row, row < N);
  for (; row < N; row += stride) {
    Raw nxt;
    request(nxt, row + stride, row + stride < N);
    const RowWindow<T> w(x + row * C, C);
    const int tail_slot = (w.packets - 1) / kTPR, tail_lane = (w.packets - 1) % kTPR;
    const bool head_partial = w.lead > 0 || (w.packets == 1 && w.tail_valid < kVec);
    const bool tail_partial = w.packets > 1 && w.tail_valid < kVec;
    auto keep = [&](u32x4& packet, const int first, const int last) {
      A v[kVec];
      IO<T>::unpack(packet, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < first || e >= last) v[e] = acc_neg_inf<A>();
      }
      packet = IO<T>::pack(v);
    };
    if (head_partial && lane == 0) keep(cur.p[0], w.lead, w.packets == 1 ? w.tail_valid : kVec);
    if (tail_partial && lane == tail_lane) {
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (i == tail_slot) keep(cur.p[i], 0, w.tail_valid);
      }
    }
    Tile t;
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      cur.unpack(i, t.v[i]);
      const bool on = Tile::active(i, w.packets);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = on ? t.v[i][e] : acc_neg_inf<A>();  // raw padding is zero bits
        m = MaxOp()(m, t.v[i][e]);
      }
    }
    m = Tile::reduce(m, MaxOp(), slots[0]);
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (kKind == kSoftmax) {
          t.v[i][e] = M::exp_of(t.v[i][e] - m);
          s += t.v[i][e];
        } else {
          t.v[i][e] = t.v[i][e] - m;
          s += M::exp_of(t.v[i][e]);
        }
      }
    s = Tile::reduce(s, SumOp(), slots[1]);
    const A inv = A(1) / s;
    const A l = acc_log(s);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = kKind == kSoftmax ? M::normalise(t.v[i][e], s, inv) : t.v[i][e] - l;
      }
    nxt.wait_ready();
    cur = nxt;
    T* base = y + row * C - w.lead;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int idx = i * kTPR + lane;
      if (idx < w.packets) {
        const u32x4 packet = IO<T>::pack(t.v[i]);
        if (idx == 0 && head_partial) {
          edge[0] = packet;
        } else if (idx == w.packets - 1 && tail_partial) {
          edge[1] = packet;
        } else {
          store_packet(base + static_cast<int64_t>(idx) * kVec, packet);
        }
      }
    }
    __syncthreads();  // slots are reused by the next row; the edge packets are in LDS
    if (lane < 2 * kVec) {
      const int which = lane / kVec, e = lane % kVec;
      const T* from = reinterpret_cast<const T*>(&edge[which]);
      if (which == 0 && head_partial) {
        const int last = w.packets == 1 ? w.tail_valid : kVec;
        if (e >= w.lead && e < last) base[e] = from[e];
      } else if (which == 1 && tail_partial) {
        if (e < w.tail_valid) base[static_cast<int64_t>(w.packets - 1) * kVec + e] = from[e];
      }
    }
  }
}

// 16-bit rows of 4097 to 8192 packets that are not whole aligned packets (a
// 50257-entry vocabulary), through their windows like softmax_wide_windows:
// eight packets per thread of a 1024-thread workgroup do not leave room for
// their 64 converted elements beside the next row's packets, so the row stays
// in raw packets, which are converted in each of the three passes (the
// exponential is taken twice), and the next row is requested ahead.
template <typename T, int kKind>
__global__ __launch_bounds__(1024) void softmax_wide_raw_windows(const int64_t N, const int C,
                                                                 const T* x, T* y) {
  constexpr int kTPR = 1024, kVPT = 8;
  using Tile = RowTile<T, kTPR, kVPT, kTPR, false>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  __shared__ u32x4 edge[2];
  const int lane = threadIdx.x;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  auto request = [&](Raw& t, const int64_t at, const bool valid) {
    const int64_t from = valid ? at : 0;
    const RowWindow<T> w(x + from * C, C);
    t.load(x + from * C - w.lead, w.packets, valid);
  };
  Raw cur;
  request(cur, row, row < N);
  for (; row < N; row += stride) {
    Raw nxt;
    request(nxt, row + stride, row + stride < N);
    const RowWindow<T> w(x + row * C, C);
    const int tail_slot = (w.packets - 1) / kTPR, tail_lane = (w.packets - 1) % kTPR;
    const bool head_partial = w.lead > 0 || (w.packets == 1 && w.tail_valid < kVec);
    const bool tail_partial = w.packets > 1 && w.tail_valid < kVec;
    auto keep = [&](u32x4& packet, const int first, const int last) {
      A v[kVec];
      IO<T>::unpack(packet, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < first || e >= last) v[e] = acc_neg_inf<A>();
      }
      packet = IO<T>::pack(v);
    };
    if (head_partial && lane == 0) keep(cur.p[0], w.lead, w.packets == 1 ? w.tail_valid : kVec);
    if (tail_partial && lane == tail_lane) {
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (i == tail_slot) keep(cur.p[i], 0, w.tail_valid);
      }
    }
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A v[kVec];
      cur.unpack(i, v);
      if (Tile::active(i, w.packets)) {  // slots beyond the window hold zero bits
#pragma unroll
        for (int e = 0; e < kVec; ++e) m = MaxOp()(m, v[e]);
      }
    }
    m = Tile::reduce(m, MaxOp(), slots[0]);
    cur.refresh();
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A v[kVec];
      cur.unpack(i, v);
      if (Tile::active(i, w.packets)) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) s += M::exp_of(v[e] - m);  // exp(-inf) = 0 beside the row
      }
    }
    s = Tile::reduce(s, SumOp(), slots[1]);
    cur.refresh();
    const A inv = A(1) / s;
    const A l = acc_log(s);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A v[kVec];
      cur.unpack(i, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const A d = v[e] - m;
        v[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), s, inv) : d - l;
      }
      cur.p[i] = IO<T>::pack(v);
    }
    nxt.wait_ready();
    T* base = y + row * C - w.lead;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int idx = i * kTPR + lane;
      if (idx < w.packets) {
        if (idx == 0 && head_partial) {
          edge[0] = cur.p[i];
        } else if (idx == w.packets - 1 && tail_partial) {
          edge[1] = cur.p[i];
        } else {
          store_packet(base + static_cast<int64_t>(idx) * kVec, cur.p[i]);
        }
      }
    }
    cur = nxt;
    __syncthreads();  // slots are reused by the next row; the edge packets are in LDS
    if (lane < 2 * kVec) {
      const int which = lane / kVec, e = lane % kVec;
      const T* from = reinterpret_cast<const T*>(&edge[which]);
      if (which == 0 && head_partial) {
        const int last = w.packets == 1 ? w.tail_valid : kVec;
        if (e >= w.lead && e < last) base[e] = from[e];
      } else if (which == 1 && tail_partial) {
        if (e < w.tail_valid) base[static_cast<int64_t>(w.packets - 1) * kVec + e] = from[e];
      }
    }
  }
}

template <typename T, int kKind, int kTPR, int kVPT, bool kRagged, bool kWindow = false>
__global__ __launch_bounds__(row_threads(kTPR)) void softmax_grad_rows(
    const int64_t N, const int C, const T* dy, const T* y, T* dx) {
  static_assert(!(kWindow && kRagged), "windows use the regular tile");
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[Tile::kSlots];
  const int npackets = Tile::extent_of(C);

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < N; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile g, o;
    const RowWindow<T> w(dy + row * C, C);  // the same for y and dx: congruent tensors
    if constexpr (kWindow) {
      g.load_window(dy + row * C, w, A(0));
      o.load_window(y + row * C, w, kKind == kSoftmax ? A(0) : acc_neg_inf<A>());
    } else {
      g.load(dy + row * C, npackets, A(0));
      o.load(y + row * C, npackets, kKind == kSoftmax ? A(0) : acc_neg_inf<A>());
    }

    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (kKind == kSoftmax) {
          s += g.v[i][e] * o.v[i][e];
        } else {
          s += g.v[i][e];
        }
      }
    s = Tile::reduce(s, SumOp(), slots);

#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (kKind == kSoftmax) {
          g.v[i][e] = (g.v[i][e] - s) * o.v[i][e];
        } else {
          g.v[i][e] = g.v[i][e] - M::exp_of(o.v[i][e]) * s;
        }
      }
    if constexpr (kWindow) {
      g.store_window(dx + row * C, w);
    } else {
      g.store(dx + row * C, npackets);
    }
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// Rows of up to 16384 packets (a 128K-entry 16-bit or a 64K-entry fp32
// vocabulary): sixteen raw packets per thread of a 1024-thread workgroup, any
// width and alignment. One read of x; fp32 / fp64 packets keep the
// exponentials in place, 16-bit packets evaluate them twice.
template <typename T, int kKind, bool kRagged>
__global__ __launch_bounds__(1024) void softmax_huge_rows(const int64_t N, const int C, const T* x,
                                                          T* y) {
  constexpr int kTPR = 1024, kVPT = 16;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Raw::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Raw::kVec;
  constexpr bool kKeepExp = kKind == kSoftmax && sizeof(T) == sizeof(A);
  __shared__ A slots[2][kTPR / kWaveSize];
  const int lane = threadIdx.x;
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    Raw t;
    if (kRagged) {
      t.load_any(x + row * C, C);
    } else {
      t.load(x + row * C, C / kVec);
    }
    // whether element e of slot i lies inside the row (regular rows: whole packets)
    auto inside = [&](int i, int e) {
      const int col = (i * kTPR + lane) * kVec;
      return kRagged ? col + e < C : col < C;
    };
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A v[kVec];
      t.unpack(i, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (inside(i, e)) m = MaxOp()(m, v[e]);
      }
    }
    m = block_allreduce<kTPR / kWaveSize>(m, MaxOp(), slots[0]);
    t.refresh();
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A v[kVec];
      t.unpack(i, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        v[e] = inside(i, e) ? M::exp_of(v[e] - m) : A(0);
        s += v[e];
      }
      if (kKeepExp) t.p[i] = IO<T>::pack(v);
    }
    s = block_allreduce<kTPR / kWaveSize>(s, SumOp(), slots[1]);
    t.refresh();
    const A inv = A(1) / s;
    const A l = acc_log(s);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int col = (i * kTPR + lane) * kVec;
      if (col < C) {
        A v[kVec];
        t.unpack(i, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (kKeepExp) {
            v[e] = M::normalise(v[e], s, inv);
          } else {
            const A d = v[e] - m;
            v[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), s, inv) : d - l;
          }
        }
        if (!kRagged) {
          store_packet(y + row * C + col, IO<T>::pack(v));
        } else if (col + kVec <= C) {
          store_packet_unaligned(y + row * C + col, IO<T>::pack(v));
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (col + e < C) IO<T>::store1(y + row * C + col + e, v[e]);
          }
        }
      }
    }
    __syncthreads();  // slots are reused by the next row
  }
}

// The gradient for 1024-thread rows: dy and y as raw packets, the next row
// prefetched where two rows of packets fit the registers (kPrefetch).
template <typename T, int kKind, int kVPT, bool kPrefetch>
__global__ __launch_bounds__(1024) void softmax_grad_wide_rows(const int64_t N, const int C,
                                                               const T* dy, const T* y, T* dx) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[Tile::kSlots];
  const int npackets = C / kVec;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  Raw tg, to;
  if (kPrefetch) {
    tg.load(dy + (row < N ? row : 0) * C, npackets, row < N);
    to.load(y + (row < N ? row : 0) * C, npackets, row < N);
  }
  for (; row < N; row += stride) {
    Raw ng, no;
    if (kPrefetch) {
      const bool more = row + stride < N;
      ng.load(dy + (more ? row + stride : 0) * C, npackets, more);
      no.load(y + (more ? row + stride : 0) * C, npackets, more);
    } else {
      tg.load(dy + row * C, npackets);
      to.load(y + row * C, npackets);
    }
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A g[kVec], o[kVec];
      tg.unpack(i, g);
      to.unpack(i, o);
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += kKind == kSoftmax ? g[e] * o[e] : g[e];  // padding: dy = 0
    }
    s = Tile::reduce(s, SumOp(), slots);
    tg.refresh();
    to.refresh();
    u32x4 out[kVPT];
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A g[kVec], o[kVec];
      tg.unpack(i, g);
      to.unpack(i, o);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        g[e] = kKind == kSoftmax ? (g[e] - s) * o[e] : g[e] - M::exp_of(o[e]) * s;
      }
      out[i] = IO<T>::pack(g);
    }
    if (kPrefetch) {
      ng.wait_ready();
      no.wait_ready();
    }
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        store_packet(dx + row * C + static_cast<int64_t>(i * kTPR + threadIdx.x) * kVec, out[i]);
      }
    }
    if (kPrefetch) tg = ng, to = no;
    __syncthreads();  // slots are reused by the next row
  }
}

// softmax_grad_wide_rows for rows that are not whole aligned packets, through
// their windows: dy, y and dx must be congruent modulo 16 bytes. A window may be
// one packet longer than the row has whole packets: the caller picks kVPT for
// C / kVec + 2 packets. Without it such rows take two passes over dy and y.
template <typename T, int kKind, int kVPT, bool kPrefetch>
__global__ __launch_bounds__(1024) void softmax_grad_wide_windows(const int64_t N, const int C,
                                                                  const T* dy, const T* y, T* dx) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[Tile::kSlots];
  __shared__ u32x4 edge[2];
  const int lane = threadIdx.x;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  auto request = [&](Raw& g, Raw& o, const int64_t at, const bool valid) {
    const int64_t from = valid ? at : 0;
    const RowWindow<T> w(dy + from * C, C);
    g.load(dy + from * C - w.lead, w.packets, valid);
    o.load(y + from * C - w.lead, w.packets, valid);
  };
  Raw tg, to;
  if (kPrefetch) request(tg, to, row, row < N);
  for (; row < N; row += stride) {
    Raw ng, no;
    if (kPrefetch) {
      request(ng, no, row + stride, row + stride < N);
    } else {
      request(tg, to, row, true);
    }
    const RowWindow<T> w(dy + row * C, C);
    const int tail_slot = (w.packets - 1) / kTPR, tail_lane = (w.packets - 1) % kTPR;
    const bool head_partial = w.lead > 0 || (w.packets == 1 && w.tail_valid < kVec);
    const bool tail_partial = w.packets > 1 && w.tail_valid < kVec;
    // What the window's first and last packet hold of the neighbouring rows is zeroed in
    // the two lanes concerned before the row is summed (slots beyond the window hold zero
    // bits already), so the passes below are those of rows of whole packets.
    auto keep = [&](u32x4& packet, const int first, const int last) {
      A v[kVec];
      IO<T>::unpack(packet, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < first || e >= last) v[e] = A(0);
      }
      packet = IO<T>::pack(v);
    };
    if (head_partial && lane == 0) {
      const int last = w.packets == 1 ? w.tail_valid : kVec;
      keep(tg.p[0], w.lead, last);
      keep(to.p[0], w.lead, last);
    }
    if (tail_partial && lane == tail_lane) {
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (i == tail_slot) {
          keep(tg.p[i], 0, w.tail_valid);
          keep(to.p[i], 0, w.tail_valid);
        }
      }
    }
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A g[kVec], o[kVec];
      tg.unpack(i, g);
      to.unpack(i, o);
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += kKind == kSoftmax ? g[e] * o[e] : g[e];
    }
    s = Tile::reduce(s, SumOp(), slots);
    tg.refresh();
    to.refresh();
    // the results replace the packets of dy: no third set of registers
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A g[kVec], o[kVec];
      tg.unpack(i, g);
      to.unpack(i, o);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        g[e] = kKind == kSoftmax ? (g[e] - s) * o[e] : g[e] - M::exp_of(o[e]) * s;
      }
      tg.p[i] = IO<T>::pack(g);
    }
    if (kPrefetch) {
      ng.wait_ready();
      no.wait_ready();
    }
    // Whole packets of the row are stored as they are; the window's first and last
    // packet, when they also hold elements of the neighbouring rows, go through LDS
    // and are stored element by element by the first threads of the workgroup.
    T* base = dx + row * C - w.lead;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int idx = i * kTPR + lane;
      if (idx < w.packets) {
        if (idx == 0 && head_partial) {
          edge[0] = tg.p[i];
        } else if (idx == w.packets - 1 && tail_partial) {
          edge[1] = tg.p[i];
        } else {
          store_packet(base + static_cast<int64_t>(idx) * kVec, tg.p[i]);
        }
      }
    }
    if (kPrefetch) tg = ng, to = no;
    __syncthreads();  // slots are reused by the next row; the edge packets are in LDS
    if (lane < 2 * kVec) {
      const int which = lane / kVec, e = lane % kVec;
      const T* from = reinterpret_cast<const T*>(&edge[which]);
      if (which == 0 && head_partial) {
        const int last = w.packets == 1 ? w.tail_valid : kVec;
        if (e >= w.lead && e < last) base[e] = from[e];
      } else if (which == 1 && tail_partial) {
        if (e < w.tail_valid) base[static_cast<int64_t>(w.packets - 1) * kVec + e] = from[e];
      }
    }
  }
}

// S > 1 with the whole reduced axis in one register tile (col_tile.h): every
// tensor is read once. 16-bit types evaluate the exponential twice (statistics
// and output) instead of keeping fp32 copies of the tile.
// With a Gather, the thread that holds the class a position's target names
// also writes that position's loss and mask (SparseCrossEntropy folded in).
struct NoGather {
  static constexpr bool kOn = false;
};
template <typename T, typename TargetT>
struct LossGather {
  static constexpr bool kOn = true;
  int64_t ignore_index;
  const TargetT* target;  // [N, S]
  T* loss;                // [N, S]
  T* mask;
};

template <typename T, int kKind, int kTW, int kR, typename Gather = NoGather>
__global__ __launch_bounds__(kColThreads) void softmax_col_tiles(const ColGrid g, const T* x, T* y,
                                                                 const Gather gather = Gather()) {
  using Tile = ColTile<T, kTW, kR>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  // Up to 8 packets per thread are converted once and held as accumulator
  // values; longer tiles stay raw packets and are converted in every pass.
  constexpr bool kHold = kR <= 8;
  // The exponentials of the statistics pass are kept where the tile holds
  // accumulator-typed values (held tiles; raw fp32 / fp64 packets); raw 16-bit
  // packets evaluate them again for the output.
  constexpr bool kKeepExp = kKind == kSoftmax && (kHold || sizeof(T) == sizeof(A));
  __shared__ A lds[Tile::kLdsWords];
  __shared__ int wanted_lds[Gather::kOn ? kTW * kVec : 1];
  __shared__ A picked_lds[Gather::kOn ? kTW * kVec : 1];
  const int nr = Tile::rows_used(g.C);  // uniform: later packets are padding
  for (int64_t tile = blockIdx.x; tile < g.tiles; tile += gridDim.x) {
    const int64_t n = tile / g.strips;
    const int64_t s0 = (tile - n * g.strips) * Tile::kCols + Tile::tw() * kVec;
    const int64_t left = g.S - s0;
    const int nvalid = left >= kVec ? kVec : (left > 0 ? static_cast<int>(left) : 0);
    const int64_t base = n * g.C * g.S + (nvalid > 0 ? s0 : 0);
    Tile t;
    t.load(x + base, g.S, g.C, nvalid, acc_neg_inf<A>());
    // Gather: the class whose probability is a column's loss (-1: none). The
    // threads of the first row group read the targets and pass them to the
    // others of their columns through LDS, so that a target is requested once.
    int wanted[kVec];
    if constexpr (Gather::kOn) {
      if (Tile::tc() == 0) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          wanted[e] = -1;
          if (e < nvalid) {
            const auto tgt = gather.target[n * g.S + s0 + e];
            if (target_valid(tgt, gather.ignore_index, g.C)) wanted[e] = static_cast<int>(tgt);
          }
        }
      }
    }
    A held[kHold ? kR : 1][kVec];
    if constexpr (kHold) {
#pragma unroll
      for (int r = 0; r < kR; ++r) t.unpack(r, held[r]);
    }
    auto get = [&](int r, A(&v)[kVec]) {
      if constexpr (kHold) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = held[r][e];
      } else {
        t.unpack(r, v);
      }
    };
    auto put = [&](int r, const A(&v)[kVec]) {
      if constexpr (kHold) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) held[r][e] = v[e];
      } else {
        t.set(r, v);
      }
    };
    A m[kVec], sum[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) m[e] = acc_neg_inf<A>(), sum[e] = A(0);
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A v[kVec];
        get(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) m[e] = MaxOp()(m[e], v[e]);
      }
    }
    Tile::reduce_rows(m, MaxOp(), lds);
    if constexpr (Gather::kOn) {
      // after that reduction's barriers (every thread is done with the previous
      // tile's values), read after the next reduction's
      if (Tile::tc() == 0) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) wanted_lds[Tile::tw() * kVec + e] = wanted[e];
      }
    }
    if (!kHold) t.refresh();
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A v[kVec];
        get(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          v[e] = kKind == kSoftmax ? M::exp_of(v[e] - m[e]) : v[e] - m[e];  // padding: exp(-inf) = 0
          sum[e] += kKind == kSoftmax ? v[e] : M::exp_of(v[e]);
        }
        if (kKeepExp || (kHold && kKind == kLogSoftmax)) put(r, v);
      }
    }
    Tile::reduce_rows(sum, SumOp(), lds);
    if (!kHold) t.refresh();
    A inv[kVec], l[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) inv[e] = A(1) / sum[e], l[e] = acc_log(sum[e]);
    A picked[kVec];      // Gather: the target class's probability where this thread holds it
    unsigned found = 0;  // one bit per column
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      picked[e] = A(0);
      if constexpr (Gather::kOn) wanted[e] = wanted_lds[Tile::tw() * kVec + e];
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A v[kVec];
        get(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (kKeepExp) {
            v[e] = M::normalise(v[e], sum[e], inv[e]);
          } else if (kHold) {  // log-softmax: the held value is x - max
            v[e] = v[e] - l[e];
          } else {
            const A d = v[e] - m[e];
            v[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), sum[e], inv[e]) : d - l[e];
          }
        }
        Tile::store(y + base, g.S, g.C, nvalid, r, v);
        if constexpr (Gather::kOn) {
          // kept in registers until the tile is done: a store per row and column
          // would be a vector-memory instruction with a lane or two active
          const int c = r * Tile::kTC + Tile::tc();
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (c == wanted[e]) picked[e] = v[e], found |= 1u << e;  // wanted < C: never padding
          }
        }
      }
    }
    if constexpr (Gather::kOn) {
      // The probabilities go back to the first row group, which writes loss and
      // mask as whole packets (a store from wherever the class was held would
      // touch every cache line of the two arrays four times, a few bytes each).
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (found & (1u << e)) picked_lds[Tile::tw() * kVec + e] = picked[e];
      }
      __syncthreads();
      if (Tile::tc() == 0 && nvalid > 0) {
        A lv[kVec], mv[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const bool on = wanted[e] >= 0;
          lv[e] = on ? neg_log_clamped(picked_lds[Tile::tw() * kVec + e]) : A(0);
          mv[e] = on ? A(1) : A(0);
        }
        T* lp = gather.loss + n * g.S + s0;
        T* mp = gather.mask + n * g.S + s0;
        const bool whole = ((reinterpret_cast<uintptr_t>(lp) | reinterpret_cast<uintptr_t>(mp)) & 15u) == 0;
        if (nvalid == kVec && whole) {
          store_packet(lp, IO<T>::pack(lv));
          store_packet(mp, IO<T>::pack(mv));
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (e < nvalid) lp[e] = lv[e], mp[e] = mv[e];
          }
        }
      }
    }
  }
}

template <typename T, int kKind, int kTW, int kR>
__global__ __launch_bounds__(kColThreads) void softmax_grad_col_tiles(const ColGrid g,
                                                                      const T* dy, const T* y,
                                                                      T* dx) {
  using Tile = ColTile<T, kTW, kR>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  __shared__ A lds[Tile::kLdsWords];
  const int nr = Tile::rows_used(g.C);  // uniform: later packets are padding
  for (int64_t tile = blockIdx.x; tile < g.tiles; tile += gridDim.x) {
    const int64_t n = tile / g.strips;
    const int64_t s0 = (tile - n * g.strips) * Tile::kCols + Tile::tw() * kVec;
    const int64_t left = g.S - s0;
    const int nvalid = left >= kVec ? kVec : (left > 0 ? static_cast<int>(left) : 0);
    const int64_t base = n * g.C * g.S + (nvalid > 0 ? s0 : 0);
    Tile tg, to;
    tg.load(dy + base, g.S, g.C, nvalid, A(0));
    to.load(y + base, g.S, g.C, nvalid, kKind == kSoftmax ? A(0) : acc_neg_inf<A>());
    A sum[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) sum[e] = A(0);
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A gv[kVec], ov[kVec];
        tg.unpack(r, gv);
        to.unpack(r, ov);
#pragma unroll
        for (int e = 0; e < kVec; ++e) sum[e] += kKind == kSoftmax ? gv[e] * ov[e] : gv[e];
      }
    }
    Tile::reduce_rows(sum, SumOp(), lds);
    tg.refresh();
    to.refresh();
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A gv[kVec], ov[kVec];
        tg.unpack(r, gv);
        to.unpack(r, ov);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          gv[e] = kKind == kSoftmax ? (gv[e] - sum[e]) * ov[e] : gv[e] - M::exp_of(ov[e]) * sum[e];
        }
        Tile::store(dx + base, g.S, g.C, nvalid, r, gv);
      }
    }
  }
}

// S > 1 with a reduced axis too long for a register tile (more than 1024
// classes): a workgroup owns a panel of all C rows by kTW * kVec adjacent
// columns of one n and walks it in chunks of ColTile::kMaxC rows, twice. Pass
// one keeps, per thread and column, a running maximum and a sum rescaled to it;
// the row threads of a column are then combined once. Pass two reads the
// chunks again (from the caches where the panel fits them), normalises and
// writes. Each chunk is read before it is written, so y may alias x.
constexpr int kPanelPackets = 8;  // packets per thread and chunk

template <typename T, int kKind, int kTW>
__global__ __launch_bounds__(kColThreads) void softmax_col_panels(const ColGrid g, const T* x,
                                                                  T* y) {
  using Tile = ColTile<T, kTW, kPanelPackets>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  constexpr int kR = kPanelPackets;
  __shared__ A lds[Tile::kLdsWords];
  for (int64_t tile = blockIdx.x; tile < g.tiles; tile += gridDim.x) {
    const int64_t n = tile / g.strips;
    const int64_t s0 = (tile - n * g.strips) * Tile::kCols + Tile::tw() * kVec;
    const int64_t left = g.S - s0;
    const int nvalid = left >= kVec ? kVec : (left > 0 ? static_cast<int>(left) : 0);
    const int64_t base = n * g.C * g.S + (nvalid > 0 ? s0 : 0);
    A m[kVec], sum[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) m[e] = acc_neg_inf<A>(), sum[e] = A(0);
    for (int c0 = 0; c0 < g.C; c0 += Tile::kMaxC) {
      Tile t;
      t.load(x + base + static_cast<int64_t>(c0) * g.S, g.S, g.C - c0, nvalid, acc_neg_inf<A>());
      A pm[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) pm[e] = acc_neg_inf<A>();
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        A v[kVec];
        t.unpack(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) pm[e] = MaxOp()(pm[e], v[e]);
      }
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (pm[e] > m[e]) {
          sum[e] *= M::exp_of(m[e] - pm[e]);  // m == -inf so far: the sum is 0 and stays 0
          m[e] = pm[e];
        }
      }
      t.refresh();
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        A v[kVec];
        t.unpack(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (m[e] > acc_neg_inf<A>()) sum[e] += M::exp_of(v[e] - m[e]);  // padding: exp(-inf) = 0
        }
      }
    }
    A top[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) top[e] = m[e];
    Tile::reduce_rows(top, MaxOp(), lds);
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      sum[e] = m[e] > acc_neg_inf<A>() ? sum[e] * M::exp_of(m[e] - top[e]) : A(0);
    }
    Tile::reduce_rows(sum, SumOp(), lds);
    A inv[kVec], l[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) inv[e] = A(1) / sum[e], l[e] = acc_log(sum[e]);
    for (int c0 = 0; c0 < g.C; c0 += Tile::kMaxC) {
      const int64_t at = base + static_cast<int64_t>(c0) * g.S;
      Tile t;
      t.load(x + at, g.S, g.C - c0, nvalid, acc_neg_inf<A>());
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        A v[kVec];
        t.unpack(r, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A d = v[e] - top[e];
          v[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), sum[e], inv[e]) : d - l[e];
        }
        Tile::store(y + at, g.S, g.C - c0, nvalid, r, v);
      }
    }
  }
}

// The backward of the same panels: pass one sums dy * y (softmax) or dy
// (log-softmax) over C, pass two reads both tensors again. dx may alias dy.
template <typename T, int kKind, int kTW>
__global__ __launch_bounds__(kColThreads) void softmax_grad_col_panels(const ColGrid g, const T* dy,
                                                                       const T* y, T* dx) {
  using Tile = ColTile<T, kTW, kPanelPackets>;
  using A = typename Tile::A;
  using M = SoftmaxMath<T>;
  constexpr int kVec = Tile::kVec;
  constexpr int kR = kPanelPackets;
  __shared__ A lds[Tile::kLdsWords];
  const A y_fill = kKind == kSoftmax ? A(0) : acc_neg_inf<A>();
  for (int64_t tile = blockIdx.x; tile < g.tiles; tile += gridDim.x) {
    const int64_t n = tile / g.strips;
    const int64_t s0 = (tile - n * g.strips) * Tile::kCols + Tile::tw() * kVec;
    const int64_t left = g.S - s0;
    const int nvalid = left >= kVec ? kVec : (left > 0 ? static_cast<int>(left) : 0);
    const int64_t base = n * g.C * g.S + (nvalid > 0 ? s0 : 0);
    A sum[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) sum[e] = A(0);
    for (int c0 = 0; c0 < g.C; c0 += Tile::kMaxC) {
      const int64_t at = base + static_cast<int64_t>(c0) * g.S;
      Tile tg, to;
      tg.load(dy + at, g.S, g.C - c0, nvalid, A(0));
      if (kKind == kSoftmax) to.load(y + at, g.S, g.C - c0, nvalid, y_fill);
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        A gv[kVec], ov[kVec];
        tg.unpack(r, gv);
        if (kKind == kSoftmax) to.unpack(r, ov);
#pragma unroll
        for (int e = 0; e < kVec; ++e) sum[e] += kKind == kSoftmax ? gv[e] * ov[e] : gv[e];
      }
    }
    Tile::reduce_rows(sum, SumOp(), lds);
    for (int c0 = 0; c0 < g.C; c0 += Tile::kMaxC) {
      const int64_t at = base + static_cast<int64_t>(c0) * g.S;
      Tile tg, to;
      tg.load(dy + at, g.S, g.C - c0, nvalid, A(0));
      to.load(y + at, g.S, g.C - c0, nvalid, y_fill);
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        A gv[kVec], ov[kVec];
        tg.unpack(r, gv);
        to.unpack(r, ov);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          gv[e] = kKind == kSoftmax ? (gv[e] - sum[e]) * ov[e] : gv[e] - M::exp_of(ov[e]) * sum[e];
        }
        Tile::store(dx + at, g.S, g.C - c0, nvalid, r, gv);
      }
    }
  }
}

// Threads along the columns of a panel: the widest of 64 / 16 / 4 that the
// columns fill and that still gives every compute unit a couple of panels.
inline int pick_panel_tw(int64_t N, int64_t S, int vec) {
  const int64_t packets = ceil_div(S, vec);
  const int tw_cap = packets > 16 ? 64 : (packets > 4 ? 16 : 4);
  for (int tw : {64, 16}) {
    if (tw > tw_cap) continue;
    if (N * ceil_div(S, static_cast<int64_t>(tw) * vec) >= 2 * num_cus()) return tw;
  }
  return 4;
}

// One thread per (n, s) column, elements S apart.
template <typename T, int kKind>
__global__ __launch_bounds__(256) void softmax_columns(
    const int64_t N, const int64_t S, const int64_t C, const T* x, T* y) {
  using A = typename IO<T>::Acc;
  const int64_t total = N * S;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t base = (i / S) * C * S + (i % S);
    A m = acc_neg_inf<A>();
    for (int64_t k = 0; k < C; ++k) m = MaxOp()(m, IO<T>::load1(x + base + k * S));
    A s = A(0);
    for (int64_t k = 0; k < C; ++k) s += acc_exp(IO<T>::load1(x + base + k * S) - m);
    if (kKind == kSoftmax) {
      for (int64_t k = 0; k < C; ++k) {
        const A e = acc_exp(IO<T>::load1(x + base + k * S) - m);
        IO<T>::store1(y + base + k * S, e / s);
      }
    } else {
      const A l = acc_log(s);
      for (int64_t k = 0; k < C; ++k) {
        IO<T>::store1(y + base + k * S, (IO<T>::load1(x + base + k * S) - m) - l);
      }
    }
  }
}

template <typename T, int kKind>
__global__ __launch_bounds__(256) void softmax_grad_columns(
    const int64_t N, const int64_t S, const int64_t C, const T* dy, const T* y, T* dx) {
  using A = typename IO<T>::Acc;
  const int64_t total = N * S;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t base = (i / S) * C * S + (i % S);
    A s = A(0);
    for (int64_t k = 0; k < C; ++k) {
      const A g = IO<T>::load1(dy + base + k * S);
      s += kKind == kSoftmax ? g * IO<T>::load1(y + base + k * S) : g;
    }
    for (int64_t k = 0; k < C; ++k) {
      const A g = IO<T>::load1(dy + base + k * S);
      const A o = IO<T>::load1(y + base + k * S);
      IO<T>::store1(dx + base + k * S, kKind == kSoftmax ? (g - s) * o : g - acc_exp(o) * s);
    }
  }
}

// S == 1 rows too long for the register tiles. Pass one keeps a running
// maximum and a sum rescaled to it per thread (one extra exponential per
// packet), so the row is walked twice, not three times.
template <typename T, int kKind>
__global__ __launch_bounds__(kLoopThreads) void softmax_rows_looped(const int64_t N,
                                                                    const int64_t C, const T* x,
                                                                    T* y) {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  using Loop = RowLoop<T>;
  constexpr int kVec = Loop::kVec;
  __shared__ A slots[2][kLoopWaves];
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const T* xr = x + row * C;
    T* yr = y + row * C;
    A m = acc_neg_inf<A>(), s = A(0);
    Loop::visit(xr, C, acc_neg_inf<A>(), [&](int64_t, const A(&v)[kVec], int) {
      A pm = v[0];
#pragma unroll
      for (int e = 1; e < kVec; ++e) pm = MaxOp()(pm, v[e]);
      if (pm > m) {
        s *= M::exp_of(m - pm);  // m == -inf on the first finite packet: s is 0 and stays 0
        m = pm;
      }
      if (m > acc_neg_inf<A>()) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) s += M::exp_of(v[e] - m);
      }
    });
    const A row_max = block_allreduce<kLoopWaves>(m, MaxOp(), slots[0]);
    s = m > acc_neg_inf<A>() ? s * M::exp_of(m - row_max) : A(0);
    s = block_allreduce<kLoopWaves>(s, SumOp(), slots[1]);
    const A inv = A(1) / s;
    const A l = acc_log(s);
    Loop::visit(xr, C, acc_neg_inf<A>(), [&](int64_t col, const A(&v)[kVec], int n) {
      A o[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const A d = v[e] - row_max;
        o[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), s, inv) : d - l;
      }
      Loop::store(yr, col, o, n);
    });
    __syncthreads();  // slots are reused by the next row
  }
}

template <typename T, int kKind>
__global__ __launch_bounds__(kLoopThreads) void softmax_grad_rows_looped(
    const int64_t N, const int64_t C, const T* dy, const T* y, T* dx) {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  using Loop = RowLoop<T>;
  constexpr int kVec = Loop::kVec;
  __shared__ A slots[kLoopWaves];
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const T* gr = dy + row * C;
    const T* yr = y + row * C;
    T* dr = dx + row * C;
    A s = A(0);
    Loop::visit2(gr, yr, C, A(0), [&](int64_t, const A(&g)[kVec], const A(&o)[kVec], int) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += kKind == kSoftmax ? g[e] * o[e] : g[e];
    });
    s = block_allreduce<kLoopWaves>(s, SumOp(), slots);
    Loop::visit2(gr, yr, C, A(0), [&](int64_t col, const A(&g)[kVec], const A(&o)[kVec], int n) {
      A r[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        r[e] = kKind == kSoftmax ? (g[e] - s) * o[e] : g[e] - M::exp_of(o[e]) * s;
      }
      Loop::store(dr, col, r, n);
    });
    __syncthreads();
  }
}

// --------------------------------------------------------------------------
// Rows of many thousands of packets (vocabulary-sized): slices of a row in the
// registers of several workgroups that exchange their partial results inside
// one kernel (slices.h), so that several workgroups per compute unit stream
// while others reduce. Forward exchanges the running (maximum, sum of
// exp(x - maximum)) of each slice, backward one sum.
// --------------------------------------------------------------------------
template <typename T>
struct OnlineSoftmaxMerge {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  static constexpr bool kIsSum = false;
  static __device__ __forceinline__ void identity(A& m, A& s) { m = acc_neg_inf<A>(), s = A(0); }
  // Both parts rescaled to the larger maximum; parts that hold only -inf add nothing.
  static __device__ __forceinline__ void merge(A& m, A& s, A m2, A s2) {
    const A top = MaxOp()(m, m2);
    if (top > acc_neg_inf<A>()) s = s * M::exp_of(m - top) + s2 * M::exp_of(m2 - top);
    m = top;
  }
};

// A thread first takes the maximum of all its packets, then adds exp(x - that
// maximum): one exp per element instead of a rescaled running sum per packet.
// Softmax of accumulator-typed elements keeps those exponentials in the
// packets, and the second pass only scales them by exp(thread maximum - row
// maximum) / sum (fp32 exp is a dozen instructions: recomputing it made the
// kernel arithmetic-bound).
template <typename T, int kKind>
struct SoftmaxSlicesForward {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  using Merge = OnlineSoftmaxMerge<T>;
  static constexpr int kIn = 1;
  static constexpr bool kScanFirst = true;
  static constexpr bool kRewrites = kKind == kSoftmax && sizeof(T) == sizeof(A);
  A top;         // maximum of this thread's elements
  A m, s, inv;   // of the row; inv = 1/s (softmax) or log(s) (log-softmax)
  A scale;       // exp(top - m)
  __device__ __forceinline__ void begin(uint32_t, uint32_t, const T*) { top = acc_neg_inf<A>(); }
  template <int V>
  __device__ __forceinline__ void scan(const A (&x)[V]) {
#pragma unroll
    for (int e = 0; e < V; ++e) top = MaxOp()(top, x[e]);
  }
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t, uint32_t, const A (&x)[V], const A (&)[V],
                                             A& a, A& b) const {
    a = top;
    if (top > acc_neg_inf<A>()) {
#pragma unroll
      for (int e = 0; e < V; ++e) b += M::exp_of(x[e] - top);
    }
  }
  template <int V>
  __device__ __forceinline__ void accumulate_rewrite(A (&x)[V], A& a, A& b) const {
    a = top;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      x[e] = top > acc_neg_inf<A>() ? M::exp_of(x[e] - top) : A(0);
      b += x[e];
    }
  }
  __device__ __forceinline__ void finish(uint32_t, bool, A a, A b) {
    m = a, s = b;
    inv = kKind == kSoftmax ? A(1) / b : acc_log(b);
    scale = top > acc_neg_inf<A>() ? M::exp_of(top - a) : A(0);
  }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t, uint32_t, A (&x)[V], const A (&)[V]) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if constexpr (kRewrites) {
        x[e] = M::normalise(x[e] * scale, s, inv);
      } else {
        const A d = x[e] - m;
        x[e] = kKind == kSoftmax ? M::normalise(M::exp_of(d), s, inv) : d - inv;
      }
    }
  }
};

// in0 = dy, in1 = y.
template <typename T, int kKind>
struct SoftmaxSlicesBackward {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  using Merge = PairSum;
  static constexpr int kIn = 2;
  A s;
  __device__ __forceinline__ void begin(uint32_t, uint32_t, const T*) {}
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t, uint32_t, const A (&dy)[V], const A (&y)[V],
                                             A& a, A&) const {
#pragma unroll
    for (int e = 0; e < V; ++e) a += kKind == kSoftmax ? dy[e] * y[e] : dy[e];
  }
  __device__ __forceinline__ void finish(uint32_t, bool, A a, A) { s = a; }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t, uint32_t, A (&dy)[V], const A (&y)[V]) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      dy[e] = kKind == kSoftmax ? (dy[e] - s) * y[e] : dy[e] - M::exp_of(y[e]) * s;
    }
  }
};

// Rows beyond the persistent one-workgroup-per-row tiles (8192 packets) take
// the slice kernel when the caller provides scratch. Measured on MI355X: fp32
// rows of 128256 run at 0.62-0.69 of the HBM peak against 0.45-0.51 for the
// one-workgroup kernels, bf16 rows of 262144 at 0.67-0.68 against 0.48-0.52;
// at 8000 packets the persistent tiles are still ahead (0.70 against 0.54).
inline int64_t slice_rows_min_packets() { return 8193; }
inline SliceUnits row_units(int64_t N, int64_t C) {
  const uint32_t c = static_cast<uint32_t>(C);
  return SliceUnits{static_cast<uint32_t>(N), 1u, c, c, c};
}
template <typename T>
size_t softmax_slices_scratch(int64_t N, int64_t S, int64_t C) {
  constexpr int kVec = IO<T>::kVec;
  if (S != 1 || C % kVec != 0 || C / kVec < slice_rows_min_packets() || !fits_int32(N * C)) return 0;
  return coop_scratch_bytes<T>(row_units(N, C));
}

// --------------------------------------------------------------------------
// Short rows: policies of the LDS-staged kernel (short_rows.h).
// --------------------------------------------------------------------------
template <typename T, int kKind, int kE>
struct SoftmaxShortForwardOp {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  __device__ __forceinline__ void set_packed(bool) {}  // no per-element state: any order
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  __device__ __forceinline__ A fill0() const { return acc_neg_inf<A>(); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A*, int, int, A (&v)[kE], const A (&)[kE]) const {
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int j = 0; j < kE; ++j) m = MaxOp()(m, v[j]);
    m = group_allreduce<kL>(m, MaxOp());
    A s = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      if (kKind == kSoftmax) {
        v[j] = M::exp_of(v[j] - m);  // lanes past the row: exp(-inf) = 0
        s += v[j];
      } else {
        v[j] = v[j] - m;
        s += M::exp_of(v[j]);
      }
    }
    s = group_allreduce<kL>(s, SumOp());
    const A inv = A(1) / s;
    const A lg = acc_log(s);
#pragma unroll
    for (int j = 0; j < kE; ++j) v[j] = kKind == kSoftmax ? M::normalise(v[j], s, inv) : v[j] - lg;
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename T, int kE>
using SoftmaxShortForward = SoftmaxShortForwardOp<T, kSoftmax, kE>;
template <typename T, int kE>
using LogSoftmaxShortForward = SoftmaxShortForwardOp<T, kLogSoftmax, kE>;

// in0 = dy (overwritten with dx), in1 = y.
template <typename T, int kKind, int kE>
struct SoftmaxShortBackwardOp {
  using A = typename IO<T>::Acc;
  using M = SoftmaxMath<T>;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  __device__ __forceinline__ void set_packed(bool) {}  // no per-element state: any order
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return kKind == kSoftmax ? A(0) : acc_neg_inf<A>(); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A*, int, int, A (&g)[kE], const A (&o)[kE]) const {
    A s = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) s += kKind == kSoftmax ? g[j] * o[j] : g[j];
    s = group_allreduce<kL>(s, SumOp());
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      g[j] = kKind == kSoftmax ? (g[j] - s) * o[j] : g[j] - M::exp_of(o[j]) * s;
    }
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename T, int kE>
using SoftmaxShortBackward = SoftmaxShortBackwardOp<T, kSoftmax, kE>;
template <typename T, int kE>
using LogSoftmaxShortBackward = SoftmaxShortBackwardOp<T, kLogSoftmax, kE>;

// Which rows take the staged path. Measured on MI355X (fraction of the HBM peak,
// staged against the register tiles): rows of up to 512 bytes gain in both
// directions (bf16 [1M,64] 0.68 / 0.77 against 0.18 / 0.38, bf16 [605184,197]
// 0.71 / 0.56 against 0.27 / 0.23, fp32 [524288,128] 0.81 / 0.71 against
// 0.58 / 0.70); longer rows only forward and only when they are not whole aligned
// packets (fp16 [262144,577] 0.62 against 0.54; whole packets of 768 bytes: 0.71
// against 0.80).
inline bool use_short_rows(int64_t C, size_t elem_bytes, bool forward, const void* a,
                           const void* b) {
  if (C > 1024 || !congruent16(a, b)) return false;
  const size_t row_bytes = static_cast<size_t>(C) * elem_bytes;
  if (row_bytes <= 512) return true;
  const bool regular = row_bytes % 16 == 0 && aligned16(a);
  return forward && !regular;
}

inline unsigned flat_grid(int64_t threads_needed) {
  const int64_t want = ceil_div(threads_needed, 256);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 64;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

template <typename T, int kKind>
int launch_softmax(int64_t N, int64_t S, int64_t C, const void* x, void* y, void* scratch,
                   size_t scratch_bytes, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  {
    const size_t need = softmax_slices_scratch<T>(N, S, C);
    if (need > 0 && scratch && scratch_bytes >= need && aligned16(x) && aligned16(y)) {
      const int st = try_channel_slices<T>(row_units(N, C), SoftmaxSlicesForward<T, kKind>{}, xp, xp,
                                           yp, static_cast<A*>(scratch), stream);
      if (st != kNotApplicable) return st;
    }
  }
  ShortPlan sp;
  if (S == 1 && use_short_rows(C, sizeof(T), true, x, y) &&
      plan_short_rows(C, sizeof(T), 4, aligned16(x), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16;
    const unsigned grid = short_grid(N, sp.rows_per_chunk);
    if (kKind == kSoftmax) {
      DRAGON_HIP_SHORT_LAUNCH(T, SoftmaxShortForward, sp, lds, grid, stream, N, static_cast<int>(C),
                              xp, xp, yp, );
    } else {
      DRAGON_HIP_SHORT_LAUNCH(T, LogSoftmaxShortForward, sp, lds, grid, stream, N,
                              static_cast<int>(C), xp, xp, yp, );
    }
    return status_of_launch();
  }
  RowConfig cfg;
  if (S == 1 && pick_row_config(ceil_div(C, kVec), 8, &cfg)) {
    // rows that are whole, aligned packets take the regular tiles, any other
    // width or base address the ragged ones
    const bool regular = C % kVec == 0 && aligned16(x) && aligned16(y);
    // 1024-thread tiles: persistent workgroups that prefetch the next row
    // (not the ragged flavour of eight 16-bit packets per thread: 64 converted
    // elements beside the next row's packets do not fit 128 registers)
    // 16-bit rows beyond four packets per thread that are not whole aligned packets: raw
    // packets through windows, the next row ahead (rows of whole packets measured 4% faster
    // with their converted elements held, softmax_wide_rows below)
    if (sizeof(T) == 2 && !regular && congruent16(x, y) && C / kVec + 2 > 4 * 1024 &&
        C / kVec + 2 <= 8 * 1024) {
      if constexpr (sizeof(T) == 2) {
        note_flavour("softmax_wide_raw_windows");
        auto kernel = softmax_wide_raw_windows<T, kKind>;
        const unsigned resident = resident_grid(kernel, 1024, 0);
        const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C), xp, yp);
        return status_of_launch();
      }
    }
    // rows of 1024-thread size that are not whole aligned packets: the same through windows
    RowConfig wcfg;
    if (!regular && sizeof(T) <= 4 && congruent16(x, y) &&
        pick_row_config(C / kVec + 2, 8, &wcfg) && wcfg.tpr == 1024 &&
        !(wcfg.vpt == 8 && sizeof(T) == 2)) {
#define LAUNCH_WINDOWS(VPT)                                                                  \
  {                                                                                          \
    note_flavour("softmax_wide_windows<" #VPT ">");                                          \
    auto kernel = softmax_wide_windows<T, kKind, VPT>;                                       \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                \
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C), xp, yp); \
  }
      if (wcfg.vpt == 2) LAUNCH_WINDOWS(2) else if (wcfg.vpt == 4) LAUNCH_WINDOWS(4) else LAUNCH_WINDOWS(8)
#undef LAUNCH_WINDOWS
      return status_of_launch();
    }
    if (cfg.tpr == 1024 && (regular || (N > 1 && !(cfg.vpt == 8 && sizeof(T) == 2)))) {
      // ragged rows: all but the last here (whole packets may read past a row's
      // end), the last one through the element-exact tile below
      const int64_t rows = regular ? N : N - 1;
#define LAUNCH_WIDE(VPT)                                                                     \
  {                                                                                          \
    note_flavour(regular ? "softmax_wide_rows<" #VPT ">" : "softmax_wide_rows<" #VPT ",ragged>"); \
    auto kernel = regular ? softmax_wide_rows<T, kKind, VPT, false>                          \
                          : softmax_wide_rows<T, kKind, VPT, true>;                          \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                \
    const unsigned grid = rows < static_cast<int64_t>(resident) ? static_cast<unsigned>(rows) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, rows, static_cast<int>(C), xp, yp); \
    if (!regular) {                                                                          \
      hipLaunchKernelGGL((softmax_rows<T, kKind, 1024, VPT, true>), dim3(1), dim3(1024), 0,  \
                         stream, static_cast<int64_t>(1), static_cast<int>(C), xp + rows * C, \
                         yp + rows * C);                                                     \
    }                                                                                        \
  }
      if (cfg.vpt == 2) LAUNCH_WIDE(2) else if (cfg.vpt == 4) LAUNCH_WIDE(4) else LAUNCH_WIDE(8)
#undef LAUNCH_WIDE
      return status_of_launch();
    }
    // rows of the smaller tiles that are not whole aligned packets: through their windows
    if (RowConfig wc; !regular && congruent16(x, y) && pick_row_config(C / kVec + 2, 8, &wc) &&
                      wc.tpr < 1024) {
#define LAUNCH(TPR, VPT)                                                                     \
  {                                                                                          \
    using Tile = RowTile<T, TPR, VPT>;                                                       \
    const dim3 grid(row_grid(N, Tile::kRowsPerBlock * wave_rows_at_a_time<TPR, VPT>()));     \
    hipLaunchKernelGGL((softmax_rows<T, kKind, TPR, VPT, false, false, true>), grid,         \
                       dim3(Tile::kThreads), 0, stream, N, static_cast<int>(C), xp, yp);     \
  }
      DRAGON_HIP_ROW_SWITCH(wc, LAUNCH);
#undef LAUNCH
      return status_of_launch();
    }
#define LAUNCH(TPR, VPT)                                                                     \
  {                                                                                          \
    using Tile = RowTile<T, TPR, VPT>;                                                       \
    const dim3 grid(row_grid(N, Tile::kRowsPerBlock * wave_rows_at_a_time<TPR, VPT>()));          \
    const dim3 block(Tile::kThreads);                                                        \
    if (regular && C / kVec == TPR * VPT) {                                                  \
      hipLaunchKernelGGL((softmax_rows<T, kKind, TPR, VPT, false, true>), grid, block, 0,    \
                         stream, N, static_cast<int>(C), xp, yp);                            \
    } else if (regular) {                                                                    \
      hipLaunchKernelGGL((softmax_rows<T, kKind, TPR, VPT, false>), grid, block, 0, stream, N, \
                         static_cast<int>(C), xp, yp);                                       \
    } else {                                                                                 \
      hipLaunchKernelGGL((softmax_rows<T, kKind, TPR, VPT, true>), grid, block, 0, stream, N, \
                         static_cast<int>(C), xp, yp);                                       \
    }                                                                                        \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  } else if (S == 1 && sizeof(T) <= 4 && ceil_div(C, kVec) <= 16 * 1024) {
    const bool regular = C % kVec == 0 && aligned16(x) && aligned16(y);
    note_flavour(regular ? "softmax_huge_rows" : "softmax_huge_rows<ragged>");
    auto kernel = regular ? softmax_huge_rows<T, kKind, false> : softmax_huge_rows<T, kKind, true>;
    const unsigned resident = resident_grid(kernel, 1024, 0);
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C), xp, yp);
  } else if (S == 1) {
    hipLaunchKernelGGL((softmax_rows_looped<T, kKind>), dim3(loop_grid(N)), dim3(kLoopThreads), 0,
                       stream, N, C, xp, yp);
  } else if (const int tw = pick_col_tw(N, C, S, kVec, 16)) {
    // the widest tile wins (narrow row segments cost more than a second
    // exponential); within it, up to 8 packets per thread are held converted
    const bool small = C <= static_cast<int64_t>(kColThreads / tw) * 8;
#define LAUNCH(TW)                                                                        \
  {                                                                                       \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                  \
    const dim3 grid(col_launch_grid(g.tiles)), block(kColThreads);                        \
    if (small) {                                                                          \
      hipLaunchKernelGGL((softmax_col_tiles<T, kKind, TW, 8>), grid, block, 0, stream, g, xp, \
                         yp);                                                             \
    } else {                                                                              \
      hipLaunchKernelGGL((softmax_col_tiles<T, kKind, TW, 16>), grid, block, 0, stream, g, xp, \
                         yp);                                                             \
    }                                                                                     \
  }
    if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  } else if (C > 1024) {
    // no register tile holds the reduced axis: panels walked in chunks, twice
    const int tw = pick_panel_tw(N, S, kVec);
#define LAUNCH(TW)                                                                        \
  {                                                                                       \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                  \
    hipLaunchKernelGGL((softmax_col_panels<T, kKind, TW>), dim3(col_launch_grid(g.tiles)), \
                       dim3(kColThreads), 0, stream, g, xp, yp);                          \
  }
    if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  } else {
    hipLaunchKernelGGL((softmax_columns<T, kKind>), dim3(flat_grid(N * S)), dim3(256), 0, stream, N,
                       S, C, xp, yp);
  }
  return status_of_launch();
}

template <typename T, int kKind>
int launch_softmax_grad(int64_t N, int64_t S, int64_t C, const void* dy, const void* y, void* dx,
                        void* scratch, size_t scratch_bytes, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* gp = static_cast<const T*>(dy);
  const T* yp = static_cast<const T*>(y);
  T* dp = static_cast<T*>(dx);
  {
    const size_t need = softmax_slices_scratch<T>(N, S, C);
    if (need > 0 && scratch && scratch_bytes >= need && aligned16(dy) && aligned16(y) &&
        aligned16(dx)) {
      const int st = try_channel_slices<T>(row_units(N, C), SoftmaxSlicesBackward<T, kKind>{}, gp,
                                           yp, dp, static_cast<A*>(scratch), stream);
      if (st != kNotApplicable) return st;
    }
  }
  ShortPlan sp;
  // two staged tensors of 16 KB each: a thread has eight loads in flight while it stages
  // (4 KB each, with eight workgroups per compute unit, measured 9% slower)
  if (S == 1 && use_short_rows(C, sizeof(T), false, dy, y) && congruent16(dy, dx) &&
      plan_short_rows(C, sizeof(T), 4, aligned16(dy), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 32;
    const unsigned grid = short_grid(N, sp.rows_per_chunk);
    if (kKind == kSoftmax) {
      DRAGON_HIP_SHORT_LAUNCH(T, SoftmaxShortBackward, sp, lds, grid, stream, N,
                              static_cast<int>(C), gp, yp, dp, );
    } else {
      DRAGON_HIP_SHORT_LAUNCH(T, LogSoftmaxShortBackward, sp, lds, grid, stream, N,
                              static_cast<int>(C), gp, yp, dp, );
    }
    return status_of_launch();
  }
  RowConfig cfg;
  const bool regular = C % kVec == 0 && aligned16(dy) && aligned16(y) && aligned16(dx);
  // 1024-thread rows: raw packets, persistent workgroups; the next row is
  // prefetched up to 4 packets per thread and tensor
  if (S == 1 && regular && pick_row_config(C / kVec, 8, &cfg) && cfg.tpr == 1024) {
#define LAUNCH_WIDE(VPT, PREFETCH)                                                           \
  {                                                                                          \
    note_flavour("softmax_grad_wide_rows<" #VPT "," #PREFETCH ">");                            \
    auto kernel = softmax_grad_wide_rows<T, kKind, VPT, PREFETCH>;                           \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                \
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C), gp, yp, \
                       dp);                                                                  \
  }
    if (cfg.vpt == 2) LAUNCH_WIDE(2, true) else if (cfg.vpt == 4) LAUNCH_WIDE(4, true)
    else LAUNCH_WIDE(8, false)
#undef LAUNCH_WIDE
    return status_of_launch();
  }
  // rows of 1024-thread size that are not whole aligned packets: the same through windows
  if (S == 1 && !regular && sizeof(T) <= 4 && congruent16(dy, y) && congruent16(dy, dx) &&
      pick_row_config(C / kVec + 2, 8, &cfg) && cfg.tpr == 1024) {
#define LAUNCH_WINDOWS(VPT, PREFETCH)                                                        \
  {                                                                                          \
    note_flavour("softmax_grad_wide_windows<" #VPT "," #PREFETCH ">");                         \
    auto kernel = softmax_grad_wide_windows<T, kKind, VPT, PREFETCH>;                        \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                \
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C), gp, yp, \
                       dp);                                                                  \
  }
    if (cfg.vpt == 2) LAUNCH_WINDOWS(2, true) else if (cfg.vpt == 4) LAUNCH_WINDOWS(4, true)
    else LAUNCH_WINDOWS(8, false)
#undef LAUNCH_WINDOWS
    return status_of_launch();
  }
  // rows of the register tiles that are not whole aligned packets: through their windows
  if (S == 1 && !regular && congruent16(dy, y) && congruent16(dy, dx) &&
      pick_row_config(C / kVec + 2, 4, &cfg)) {
#define LAUNCH(TPR, VPT)                                                                     \
  {                                                                                          \
    using Tile = RowTile<T, TPR, VPT>;                                                       \
    hipLaunchKernelGGL((softmax_grad_rows<T, kKind, TPR, VPT, false, true>),                 \
                       dim3(row_grid(N, Tile::kRowsPerBlock)), dim3(Tile::kThreads), 0,      \
                       stream, N, static_cast<int>(C), gp, yp, dp);                          \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
    return status_of_launch();
  }
  // Two tiles live at once: halve the packets a thread may hold.
  if (S == 1 && pick_row_config(ceil_div(C, kVec), 4, &cfg)) {
#define LAUNCH(TPR, VPT)                                                                     \
  {                                                                                          \
    using Tile = RowTile<T, TPR, VPT>;                                                       \
    const dim3 grid(row_grid(N, Tile::kRowsPerBlock)), block(Tile::kThreads);                \
    if (regular) {                                                                           \
      hipLaunchKernelGGL((softmax_grad_rows<T, kKind, TPR, VPT, false>), grid, block, 0,     \
                         stream, N, static_cast<int>(C), gp, yp, dp);                        \
    } else {                                                                                 \
      hipLaunchKernelGGL((softmax_grad_rows<T, kKind, TPR, VPT, true>), grid, block, 0,      \
                         stream, N, static_cast<int>(C), gp, yp, dp);                        \
    }                                                                                        \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  } else if (S == 1) {
    hipLaunchKernelGGL((softmax_grad_rows_looped<T, kKind>), dim3(loop_grid(N)),
                       dim3(kLoopThreads), 0, stream, N, C, gp, yp, dp);
  } else if (const int tw = pick_col_tw(N, C, S, kVec, 16)) {
    // two tiles live at once: 8 packets per thread each where that holds C rows
    const bool small = C <= static_cast<int64_t>(kColThreads / tw) * 8;
#define LAUNCH(TW)                                                                        \
  {                                                                                       \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                  \
    const dim3 grid(col_launch_grid(g.tiles)), block(kColThreads);                        \
    if (small) {                                                                          \
      hipLaunchKernelGGL((softmax_grad_col_tiles<T, kKind, TW, 8>), grid, block, 0, stream, g, \
                         gp, yp, dp);                                                     \
    } else {                                                                              \
      hipLaunchKernelGGL((softmax_grad_col_tiles<T, kKind, TW, 16>), grid, block, 0, stream, g, \
                         gp, yp, dp);                                                     \
    }                                                                                     \
  }
    if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  } else if (C > 1024) {
    const int tw = pick_panel_tw(N, S, kVec);
#define LAUNCH(TW)                                                                          \
  {                                                                                         \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                    \
    hipLaunchKernelGGL((softmax_grad_col_panels<T, kKind, TW>), dim3(col_launch_grid(g.tiles)), \
                       dim3(kColThreads), 0, stream, g, gp, yp, dp);                        \
  }
    if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  } else {
    hipLaunchKernelGGL((softmax_grad_columns<T, kKind>), dim3(flat_grid(N * S)), dim3(256), 0,
                       stream, N, S, C, gp, yp, dp);
  }
  return status_of_launch();
}

template <typename T>
int softmax_fwd(int64_t N, int64_t S, int64_t C, const void* x, void* y, void* scratch,
                size_t scratch_bytes, hipStream_t s) {
  return launch_softmax<T, kSoftmax>(N, S, C, x, y, scratch, scratch_bytes, s);
}
template <typename T>
int log_softmax_fwd(int64_t N, int64_t S, int64_t C, const void* x, void* y, void* scratch,
                    size_t scratch_bytes, hipStream_t s) {
  return launch_softmax<T, kLogSoftmax>(N, S, C, x, y, scratch, scratch_bytes, s);
}
template <typename T>
int softmax_bwd(int64_t N, int64_t S, int64_t C, const void* dy, const void* y, void* dx,
                void* scratch, size_t scratch_bytes, hipStream_t s) {
  return launch_softmax_grad<T, kSoftmax>(N, S, C, dy, y, dx, scratch, scratch_bytes, s);
}
template <typename T>
int log_softmax_bwd(int64_t N, int64_t S, int64_t C, const void* dy, const void* y, void* dx,
                    void* scratch, size_t scratch_bytes, hipStream_t s) {
  return launch_softmax_grad<T, kLogSoftmax>(N, S, C, dy, y, dx, scratch, scratch_bytes, s);
}
template <typename T>
int softmax_scratch(int64_t N, int64_t S, int64_t C, size_t* bytes) {
  *bytes = softmax_slices_scratch<T>(N, S, C);
  return DRAGON_HIP_OK;
}

inline int check_softmax_args(int64_t N, int64_t S, int64_t C, const void* a, const void* b) {
  if (N < 0 || S < 0 || C <= 0) return DRAGON_HIP_EINVAL;
  if (N * S == 0) return 1;  // nothing to do
  if (!a || !b) return DRAGON_HIP_EINVAL;
  return 0;
}

} // namespace

template <typename T, typename TargetT>
int launch_softmax_cols_with_loss(int64_t N, int64_t S, int64_t C, int64_t ignore_index,
                                  const T* x, const TargetT* target, T* prob, T* loss, T* mask,
                                  hipStream_t stream) {
  constexpr int kVec = IO<T>::kVec;
  const int tw = pick_col_tw(N, C, S, kVec, 16);
  if (tw == 0) return 1;
  const bool small = C <= static_cast<int64_t>(kColThreads / tw) * 8;
  const LossGather<T, TargetT> gather{ignore_index, target, loss, mask};
#define LAUNCH(TW)                                                                              \
  {                                                                                             \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                        \
    const dim3 grid(col_launch_grid(g.tiles)), block(kColThreads);                              \
    if (small) {                                                                                \
      hipLaunchKernelGGL((softmax_col_tiles<T, kSoftmax, TW, 8, LossGather<T, TargetT>>), grid, \
                         block, 0, stream, g, x, prob, gather);                                 \
    } else {                                                                                    \
      hipLaunchKernelGGL((softmax_col_tiles<T, kSoftmax, TW, 16, LossGather<T, TargetT>>), grid, \
                         block, 0, stream, g, x, prob, gather);                                 \
    }                                                                                           \
  }
  if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  return status_of_launch();
}
template int launch_softmax_cols_with_loss<float, int32_t>(int64_t, int64_t, int64_t, int64_t,
                                                           const float*, const int32_t*, float*,
                                                           float*, float*, hipStream_t);
template int launch_softmax_cols_with_loss<float, int64_t>(int64_t, int64_t, int64_t, int64_t,
                                                           const float*, const int64_t*, float*,
                                                           float*, float*, hipStream_t);
template int launch_softmax_cols_with_loss<double, int32_t>(int64_t, int64_t, int64_t, int64_t,
                                                            const double*, const int32_t*, double*,
                                                            double*, double*, hipStream_t);
template int launch_softmax_cols_with_loss<double, int64_t>(int64_t, int64_t, int64_t, int64_t,
                                                            const double*, const int64_t*, double*,
                                                            double*, double*, hipStream_t);
} // namespace dragon_hip

extern "C" {

size_t dragon_hip_softmax_scratch_bytes(int dtype, int64_t N, int64_t S, int64_t C) {
  if (N <= 0 || S <= 0 || C <= 0) return 0;
  size_t bytes = 0;
  switch (dtype) {
    case DRAGON_HIP_F16: dragon_hip::softmax_scratch<dragon_hip::f16_t>(N, S, C, &bytes); break;
    case DRAGON_HIP_BF16: dragon_hip::softmax_scratch<dragon_hip::bf16_t>(N, S, C, &bytes); break;
    case DRAGON_HIP_F32: dragon_hip::softmax_scratch<float>(N, S, C, &bytes); break;
    case DRAGON_HIP_F64: dragon_hip::softmax_scratch<double>(N, S, C, &bytes); break;
    default: break;
  }
  return bytes;
}

int dragon_hip_softmax(int dtype, int64_t N, int64_t S, int64_t C, const void* x, void* y,
                       void* scratch, size_t scratch_bytes, void* stream) {
  const int c = dragon_hip::check_softmax_args(N, S, C, x, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::softmax_fwd, N, S, C, x, y, scratch, scratch_bytes, s);
}

int dragon_hip_log_softmax(int dtype, int64_t N, int64_t S, int64_t C, const void* x, void* y,
                           void* scratch, size_t scratch_bytes, void* stream) {
  const int c = dragon_hip::check_softmax_args(N, S, C, x, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::log_softmax_fwd, N, S, C, x, y, scratch,
                            scratch_bytes, s);
}

int dragon_hip_softmax_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dy,
                            const void* y, void* dx, void* scratch, size_t scratch_bytes,
                            void* stream) {
  const int c = dragon_hip::check_softmax_args(N, S, C, dy, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  if (!dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::softmax_bwd, N, S, C, dy, y, dx, scratch,
                            scratch_bytes, s);
}

int dragon_hip_log_softmax_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dy,
                                const void* y, void* dx, void* scratch, size_t scratch_bytes,
                                void* stream) {
  const int c = dragon_hip::check_softmax_args(N, S, C, dy, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  if (!dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::log_softmax_bwd, N, S, C, dy, y, dx, scratch,
                            scratch_bytes, s);
}

} // extern "C"
