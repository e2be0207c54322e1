// GroupNorm forward / backward and LayerNorm backward for gfx950.
//
// Replaces
//   kernels::GroupNorm      dragon/kernels/normalization/op_kernels.h:111-124
//                           (CPU cpu/group_norm_kernel.cc:11-31,88-110)
//   kernels::GroupNormGrad  dragon/kernels/normalization/op_kernels.h:126-143
//                           (CPU cpu/group_norm_kernel.cc:33-84,112-147)
// and, because LayerNormGradientOp is GroupNormGradientOp with G = S = 1,
// D = C and layout NHWC (dragon/operators/normalization/layer_norm_op.h:39-54),
// LayerNorm backward.
//
// x is [N, G, D, S] (NCHW) or [N, S, G, D] (NHWC); channel c = g*D + d, group
// statistics index ng = n*G + g.
//   y      = (x - mu[ng]) * rsig[ng] * gamma[c] + beta[c]
//   ds[ng] = sum gamma[c]*dy*x          db[ng] = sum gamma[c]*dy
//   dx     = gamma[c]*dy*rsig + ((db*mu - ds)*(x - mu)*rsig^3 - db*rsig) / (D*S)
//   dgamma[c] = sum dy*(x - mu[ng])*rsig[ng]    dbeta[c] = sum dy
//
// Paths
//   rows   (G = S = 1, i.e. LayerNorm backward): one fused kernel keeps x and
//          dy of a row in registers, so both are read once; dgamma/dbeta are
//          accumulated per thread across the rows a workgroup visits, combined
//          through LDS, written as one partial row per workgroup, and summed
//          by a second small kernel (two-stage, no atomics).
//   groups (NCHW, a group fits a register tile): fused forward for any S;
//          fused backward when channels span whole wavefronts of packets.
//   slices (NCHW, a group larger than one workgroup's registers): the group's
//          slices stay in the registers of several workgroups that exchange
//          their partial sums inside one kernel (slices.h), so x and dy are
//          still read once.
//   general  one pass over x and dy for the per-(n, c) pairs
//          (sum dy*(x - mu), sum dy): rows of S elements (NCHW) or column
//          reductions of each sample's [S, C] matrix (NHWC); ds/db and
//          dgamma/dbeta from those N*C pairs; one flat map for dx. Any layout,
//          any alignment.
#include <cstdlib>

#include "long_rows.h"
#include "reduce.h"
#include "row_loop.h"
#include "row_tile.h"
#include "short_rows.h"
#include "sample_slices.h"
#include "group_items.h"
#include "slices.h"

namespace dragon_hip {
namespace {

struct GroupShape {
  uint32_t N, G, D, S, C;  // C = G*D
  bool nchw;
};

// --------------------------------------------------------------------------
// Forward map
// --------------------------------------------------------------------------
// kVec consecutive per-channel parameters at p (16-byte aligned when kVec > 1:
// the packet's first channel is a multiple of kVec).
template <int kVec, typename A>
__device__ __forceinline__ void load_channel_run(const A* p, A (&v)[kVec]) {
  if constexpr (kVec == 1) {
    v[0] = p[0];
  } else {
    load_params_ragged<kVec>(p, kVec, v);
  }
}

template <typename T, int kVec>
struct GroupNormApply {
  using A = typename IO<T>::Acc;
  GroupShape sh;
  const A* mu;
  const A* rsig;
  const A* gamma;
  const A* beta;
  __device__ __forceinline__ void operator()(uint32_t i, A (&v)[kVec], const A (&)[kVec]) const {
    if (sh.nchw) {
      // A packet never straddles a row of S elements (kVec divides S or is 1).
      const uint32_t row = i / sh.S;  // = n*C + c
      const uint32_t c = row % sh.C;
      const uint32_t ng = row / sh.D;
      const A m = mu[ng];
      const A r = rsig[ng];
      const A g = gamma[c], b = beta[c];
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = (v[e] - m) * r * g + b;
    } else {
      const uint32_t c = i % sh.C;  // kVec divides C or is 1
      const uint32_t n = i / (sh.S * sh.C);
      if (kVec > 1 && sh.D % kVec == 0) {
        // the packet lies within one group: one pair of statistics, parameters as packets
        const uint32_t ng = n * sh.G + c / sh.D;
        const A m = mu[ng], r = rsig[ng];
        A g[kVec], b[kVec];
        load_params_ragged<kVec>(gamma + c, kVec, g);
        load_params_ragged<kVec>(beta + c, kVec, b);
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = (v[e] - m) * r * g[e] + b[e];
        return;
      }
      if (kVec > 1 && sh.D == 1) {
        // a group per channel: the statistics are packets as well
        A m[kVec], r[kVec], gam[kVec], bet[kVec];
        load_channel_run<kVec>(mu + n * sh.G + c, m);
        load_channel_run<kVec>(rsig + n * sh.G + c, r);
        load_channel_run<kVec>(gamma + c, gam);
        load_channel_run<kVec>(beta + c, bet);
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = (v[e] - m[e]) * r[e] * gam[e] + bet[e];
        return;
      }
      // The packet spans several groups (D is not a multiple of kVec): one
      // division per packet, then the group advances with the channel.
      uint32_t g = sh.G == 1 ? 0u : c / sh.D;
      uint32_t k = c - g * sh.D;
      A m = mu[n * sh.G + g], r = rsig[n * sh.G + g];
      A gam[kVec], bet[kVec];
      load_channel_run<kVec>(gamma + c, gam);
      load_channel_run<kVec>(beta + c, bet);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (k == sh.D) {
          k = 0, ++g;
          m = mu[n * sh.G + g], r = rsig[n * sh.G + g];
        }
        v[e] = (v[e] - m) * r * gam[e] + bet[e];
        ++k;
      }
    }
  }
};

// --------------------------------------------------------------------------
// General backward: the last step, dx from the per-group and per-row scalars
// --------------------------------------------------------------------------
template <typename T, int kVec>
struct GroupNormGradApply {
  using A = typename IO<T>::Acc;
  GroupShape sh;
  const A* mu;
  const A* rsig;
  const A* gamma;
  const A* ds;
  const A* db;
  A denom;
  __device__ __forceinline__ A one(A x, A dy, uint32_t ng, uint32_t c) const {
    const A m = mu[ng], r = rsig[ng], s = ds[ng], b = db[ng];
    const A u = (b * m - s) * (x - m) * (r * r * r);
    const A v = b * r;
    return gamma[c] * dy * r + (u - v) * denom;
  }
  __device__ __forceinline__ void operator()(uint32_t i, A (&x)[kVec], const A (&dy)[kVec]) const {
    if (sh.nchw) {
      const uint32_t row = i / sh.S;
      const uint32_t c = row % sh.C;
      const uint32_t ng = row / sh.D;
#pragma unroll
      for (int e = 0; e < kVec; ++e) x[e] = one(x[e], dy[e], ng, c);
    } else {
      const uint32_t c = i % sh.C;
      const uint32_t n = i / (sh.S * sh.C);
      if (kVec > 1 && sh.D % kVec == 0) {
        // the packet lies within one group: the group's scalars once, gamma as a packet
        const uint32_t ng = n * sh.G + c / sh.D;
        const A m = mu[ng], r = rsig[ng], s = ds[ng], b = db[ng];
        const A ku = (b * m - s) * (r * r * r) * denom;
        const A kv = b * r * denom;
        A g[kVec];
        load_params_ragged<kVec>(gamma + c, kVec, g);
#pragma unroll
        for (int e = 0; e < kVec; ++e) x[e] = g[e] * dy[e] * r + (ku * (x[e] - m) - kv);
        return;
      }
      if (kVec > 1 && sh.D == 1) {
        // a group per channel: the per-group scalars are packets as well
        A m[kVec], r[kVec], s[kVec], b[kVec], gam[kVec];
        load_channel_run<kVec>(mu + n * sh.G + c, m);
        load_channel_run<kVec>(rsig + n * sh.G + c, r);
        load_channel_run<kVec>(ds + n * sh.G + c, s);
        load_channel_run<kVec>(db + n * sh.G + c, b);
        load_channel_run<kVec>(gamma + c, gam);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A u = (b[e] * m[e] - s[e]) * (x[e] - m[e]) * (r[e] * r[e] * r[e]);
          const A v = b[e] * r[e];
          x[e] = gam[e] * dy[e] * r[e] + (u - v) * denom;
        }
        return;
      }
      // several groups per packet: as GroupNormApply
      uint32_t g = sh.G == 1 ? 0u : c / sh.D;
      uint32_t k = c - g * sh.D;
      uint32_t ng = n * sh.G + g;
      A m = mu[ng], r = rsig[ng], s = ds[ng], b = db[ng];
      A gam[kVec];
      load_channel_run<kVec>(gamma + c, gam);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (k == sh.D) {
          k = 0, ++ng;
          m = mu[ng], r = rsig[ng], s = ds[ng], b = db[ng];
        }
        const A u = (b * m - s) * (x[e] - m) * (r * r * r);
        const A v = b * r;
        x[e] = gam[e] * dy[e] * r + (u - v) * denom;
        ++k;
      }
    }
  }
};

// --------------------------------------------------------------------------
// Fused row path (LayerNorm backward)
// --------------------------------------------------------------------------

// Short rows: two 512-thread workgroups share a compute unit (128 registers per
// thread), so that one computes while the other waits for its rows. Rows of
// 2049 to 4096 elements take one 1024-thread workgroup per compute unit, which
// writes half as many partial rows. Rows of 1025 to 1536 packets take a
// 768-thread workgroup (two packets per thread, no idle lanes, 168 registers). gamma is staged in LDS once per
// (persistent) workgroup; x and dy of a row are kept as raw packets;
// dgamma / dbeta are accumulated per thread across the rows the workgroup
// visits, combined across its row groups through LDS, and written as one
// partial row per workgroup: partial[blockIdx][c][{dgamma, dbeta}].
//
// Per element, with the row scalars a = (db*mu - ds)*rsig^3/C, b = -db*rsig/C:
//   xc = x - mu;  w = dy*rsig;  dgamma += w*xc;  dbeta += dy;
//   dx = gamma*w + (a*xc + b)
// The ragged flavour takes rows of any width at element-aligned addresses:
// exact (branching) loads that zero what lies past a row, element-wise stores
// for a row's partial last packet; gamma is staged element by element.
template <typename T, int kTPR, int kVPT, int kGradThreads, bool kRagged = false>
__global__ __launch_bounds__(kGradThreads, kGradThreads == 768 ? 3 : 4) void layer_norm_grad_rows(
    const int64_t N, const int C, const T* __restrict__ x, const T* __restrict__ dy,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ mu,
    const typename IO<T>::Acc* __restrict__ rsig, typename IO<T>::Acc* __restrict__ ds,
    typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial, unsigned long long* __restrict__ stamps) {
  using Tile = RowTile<T, kTPR, kVPT, kGradThreads>;
  using Raw = RawRowTile<T, kTPR, kVPT, kGradThreads>;
  // Phase clock of this workgroup (100 MHz device clock), only when a timeline is recorded.
  unsigned long long* const mark =
      stamps != nullptr && threadIdx.x == 0 ? stamps + static_cast<size_t>(blockIdx.x) * kTimelineWords : nullptr;
  if (mark) mark[0] = wall_clock64();
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  constexpr int kGroups = Tile::kRowsPerBlock;
  constexpr int kPerPacket = 16 / sizeof(A);
  // A round of the final cross-group combine moves kChunk (dgamma, dbeta) pairs per thread.
  constexpr int kChunk = kVec < 4 ? kVec : 4;
  constexpr int kRedWords = kGroups > 1 ? (kGroups - 1) * kTPR * kChunk * 2 : 1;
  // Rows requested ahead of the current one: two where three rows of raw
  // packets and the accumulators fit the register budget (128 per thread; 168
  // for the 768-thread workgroup, which runs three wavefronts per SIMD).
  constexpr int kDepth = (kVPT * kVec <= 8 || kGradThreads == 768) ? 2 : 1;
  constexpr bool kSplit = !kRagged && kVec == 2 * kPerPacket;
  extern __shared__ u32x4 staged[];  // gamma[C]
  __shared__ A slots[2 * Tile::kSlots];
  __shared__ A red[kRedWords];
  const A* lds_gamma = reinterpret_cast<const A*>(staged);
  const int npackets_of_row = (C + kVec - 1) / kVec;
  // gamma of the kVec columns of packet `packet` of the row
  auto gamma_of = [&](const int packet, A(&g)[kVec]) {
    if constexpr (kSplit) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(lds_gamma + packet * 4);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(lds_gamma + (npackets_of_row + packet) * 4);
      g[0] = lo.x, g[1] = lo.y, g[2] = lo.z, g[3] = lo.w;
      g[4] = hi.x, g[5] = hi.y, g[6] = hi.z, g[7] = hi.w;
    } else {
      load_params<kVec>(lds_gamma + packet * kVec, g);
    }
  };
  const int npackets = (C + kVec - 1) / kVec;

  const int lane = Tile::lane();
  const int sub = Tile::sub_row();
  const A inv_c = A(1) / A(C);

  A dg[kVPT][kVec], dbt[kVPT][kVec];
#pragma unroll
  for (int i = 0; i < kVPT; ++i)
#pragma unroll
    for (int e = 0; e < kVec; ++e) dg[i][e] = dbt[i][e] = A(0);

  // The packets of the next kDepth rows are requested before the current row
  // is reduced, so their HBM latency hides behind this row's arithmetic and
  // enough bytes stay in flight per compute unit. The rows in flight live in a
  // ring of kDepth + 1 register tiles and the row loop is unrolled over the
  // ring, so that a tile never moves between registers: copying a tile whose
  // loads are in flight would wait for them. Uniform trip count across the
  // workgroup: the row reductions hold barriers.
  constexpr int kRing = kDepth + 1;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kGroups;
  int64_t row = static_cast<int64_t>(blockIdx.x) * kGroups + sub;
  // Rows past the end are clamped to row 0 for addressing; neither they nor the
  // slots beyond the row are zero-filled (no selects on the loaded packets):
  // such rows skip the second pass, and such slots only ever feed accumulators
  // of columns that are not written out.
  Raw rx[kRing], rdy[kRing];  // phase k: rx[k] is the current row, the others follow it
  A rm[kRing], rr[kRing];
  auto request = [&](Raw& tx, Raw& tdy, A& m, A& r, const int64_t at) {
    const int64_t from = at < N ? at : 0;
    if constexpr (kRagged) {
      tx.load_any(x + from * C, C);
      tdy.load_any(dy + from * C, C);
    } else {
      tx.load_unmasked(x + from * C, npackets);
      tdy.load_unmasked(dy + from * C, npackets);
    }
    m = mu[from];
    r = rsig[from];
  };
#pragma unroll
  for (int k = 0; k < kDepth; ++k) request(rx[k], rdy[k], rm[k], rr[k], row + k * stride);

  // gamma is staged while the first rows travel
  if constexpr (kRagged) {
    A* stage_gamma = reinterpret_cast<A*>(staged);
    for (int i = threadIdx.x; i < npackets * kVec; i += kGradThreads) {
      stage_gamma[i] = i < C ? gamma[i] : A(0);
    }
  } else {
    // Rows of 8-element packets against 4-float LDS words: the first halves of
    // all packets, then the second halves, so that the lanes of a wavefront read
    // adjacent 16-byte words (eight consecutive floats per lane put lanes l and
    // l + 8 on the same banks: a two-way conflict on every access).
    for (int i = threadIdx.x; i < C / kPerPacket; i += kGradThreads) {
      const int at = kSplit ? (i & 1) * npackets + (i >> 1) : i;
      staged[at] = load_packet_keep(gamma + i * kPerPacket);
    }
  }
  __syncthreads();

  unsigned long long rows_done = 0;  // of the marking thread's row group
  // One row: tx / tdy hold it, nx / ndy the row after it.
  auto step = [&](Raw& tx, Raw& tdy, const A m, const A r, Raw& nx, Raw& ndy) {
    const bool valid = row < N;
    A s1 = A(0), s2 = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        A xv[kVec], dv[kVec], g[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        gamma_of(i * kTPR + lane, g);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A t = g[e] * dv[e];
          s1 += t * xv[e];
          s2 += t;
        }
      }
    }
    Tile::reduce_sum_pair(s1, s2, slots);
    if (lane == 0 && valid) {
      ds[row] = s1;
      db[row] = s2;
    }
    if (mark && rows_done++ == 0) mark[1] = wall_clock64();  // the first row has arrived and is summed

    const A a = (s2 * m - s1) * (r * r * r) * inv_c;
    const A b = -(s2 * r) * inv_c;
    tx.refresh();
    tdy.refresh();
    u32x4 out[kVPT];
    if (valid) {  // uniform over the wavefront
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        A xv[kVec], dv[kVec], g[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        // A slot beyond the row reads gamma of column 0 .. kVec - 1: its dx is not stored.
        gamma_of(Tile::active(i, npackets) ? i * kTPR + lane : 0, g);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A xc = xv[e] - m;
          const A w = dv[e] * r;
          dg[i][e] += w * xc;
          dbt[i][e] += dv[e];
          xv[e] = g[e] * w + (a * xc + b);
        }
        out[i] = IO<T>::pack(xv);
      }
    }
    // Wait for the next row here, before this row's stores are issued (the
    // rows requested after it stay in flight).
    if (kDepth == 1) {
      nx.wait_ready();
      ndy.wait_ready();
    }
    T* dxr = dx + (valid ? row : 0) * C;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (valid && Tile::active(i, npackets)) {
        const int col = (i * kTPR + lane) * kVec;
        if constexpr (!kRagged) {
          store_packet(dxr + col, out[i]);
        } else if (col + kVec <= C) {
          store_packet_unaligned(dxr + col, out[i]);
        } else {
          A last[kVec];
          IO<T>::unpack(out[i], last);
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (col + e < C) IO<T>::store1(dxr + col + e, last[e]);
          }
        }
      }
    }
    if (Tile::kWavesPerRow > 1) __syncthreads();  // slots reused by the next row
  };

  int64_t base = static_cast<int64_t>(blockIdx.x) * kGroups;
  while (base < N) {
#pragma unroll
    for (int k = 0; k < kRing; ++k) {
      if (base < N) {  // uniform over the workgroup
        const int kFar = (k + kDepth) % kRing;  // the tile the previous row has left
        const int kNext = (k + 1) % kRing;
        request(rx[kFar], rdy[kFar], rm[kFar], rr[kFar], row + kDepth * stride);
        step(rx[k], rdy[k], rm[k], rr[k], rx[kNext], rdy[kNext]);
        row += stride;
        base += stride;
      }
    }
  }

  if (mark) mark[2] = wall_clock64();  // the row loop is done; what follows is the partial row
  // Combine the kGroups row groups of this workgroup, kChunk pairs at a time.
  A* out = partial + static_cast<size_t>(blockIdx.x) * C * 2;
#pragma unroll
  for (int i = 0; i < kVPT; ++i) {
#pragma unroll
    for (int h = 0; h < kVec / kChunk; ++h) {
      if (kGroups > 1) {
        __syncthreads();
        if (sub > 0) {
          A* w = red + (static_cast<size_t>(sub - 1) * kTPR + lane) * kChunk * 2;
#pragma unroll
          for (int e = 0; e < kChunk; ++e) {
            w[2 * e] = dg[i][h * kChunk + e];
            w[2 * e + 1] = dbt[i][h * kChunk + e];
          }
        }
        __syncthreads();
      }
      if (sub == 0 && Tile::active(i, npackets)) {
        A pg[kChunk], pb[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          pg[e] = dg[i][h * kChunk + e];
          pb[e] = dbt[i][h * kChunk + e];
        }
        for (int q = 1; q < kGroups; ++q) {
          const A* w = red + (static_cast<size_t>(q - 1) * kTPR + lane) * kChunk * 2;
#pragma unroll
          for (int e = 0; e < kChunk; ++e) {
            pg[e] += w[2 * e];
            pb[e] += w[2 * e + 1];
          }
        }
        const int col = (i * kTPR + lane) * kVec + h * kChunk;
        A* o = out + static_cast<size_t>(col) * 2;
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          if (!kRagged || col + e < C) {
            o[2 * e] = pg[e];
            o[2 * e + 1] = pb[e];
          }
        }
      }
    }
  }
  if (mark) {
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    mark[3] = wall_clock64();
    mark[4] = xcc & 0xf;
    mark[5] = rows_done;
  }
}

// --------------------------------------------------------------------------
// LayerNorm backward of short rows (per-head normalisations, odd widths): a
// policy of the LDS-staged kernel (short_rows.h). in0 = x (overwritten with
// dx), in1 = dy. A thread keeps dgamma / dbeta of its elements across the rows
// its workgroup visits; the workgroup's lane groups are combined through LDS
// into one partial row per workgroup, summed by sum_partial_rows.
// --------------------------------------------------------------------------
inline int short_grad_max_grid() { return num_cus() * 8; }

template <typename T, int kE>
struct LayerNormShortBackward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = static_cast<size_t>(kShortThreads) * kE * 2 * sizeof(A);
  static constexpr int kSideWords = 2;
  A inv_c;
  const A* mu;
  const A* rsig;
  const A* gamma;
  A* ds;
  A* db;
  A* partial;  // [gridDim.x][C][2]
  A g[kE], dg[kE], dbt[kE];
  bool packed = false;  // lane l owns elements l * kE + j instead of l + j * kL
  __device__ __forceinline__ void set_packed(bool on) { packed = on; }
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  template <int kL>
  __device__ __forceinline__ int element(int l, int j) const {
    return packed ? l * kE + j : l + j * kL;
  }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int l, int C) {
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const int e = element<kL>(l, j);
      g[j] = e < C ? gamma[e] : A(0);
      dg[j] = dbt[j] = A(0);
    }
  }
  // mean and rsig of a row: requested with the range's packets, ahead of the
  // row loop (where every row would otherwise wait for HBM)
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[2]) const {
    w[0] = mu[row];
    w[1] = rsig[row];
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t row, const A* side, int l, int, A (&x)[kE],
                                      const A (&dy)[kE]) {
    const A m = side[0], r = side[1];
    A s1 = A(0), s2 = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const A t = g[j] * dy[j];
      s1 += t * x[j];
      s2 += t;
    }
    s1 = group_allreduce<kL>(s1, SumOp());
    s2 = group_allreduce<kL>(s2, SumOp());
    if (l == 0) {
      ds[row] = s1;
      db[row] = s2;
    }
    const A a = (s2 * m - s1) * (r * r * r) * inv_c;
    const A b = -(s2 * r) * inv_c;
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const A xc = x[j] - m;
      const A w = dy[j] * r;  // lanes past the row hold dy = 0: they add nothing
      dg[j] += w * xc;
      dbt[j] += dy[j];
      x[j] = g[j] * w + (a * xc + b);
    }
  }
  template <int kL>
  __device__ __forceinline__ void end(A* lds, int C) const {
    constexpr int kGroups = kShortThreads / kL;
    const int l = threadIdx.x % kL, sub = threadIdx.x / kL;
    __syncthreads();  // the stage is free
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      lds[((sub * kE + j) * kL + l) * 2] = dg[j];
      lds[((sub * kE + j) * kL + l) * 2 + 1] = dbt[j];
    }
    __syncthreads();
    if (sub == 0) {
      A* out = partial + static_cast<size_t>(blockIdx.x) * C * 2;
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const int e = element<kL>(l, j);
        if (e < C) {
          A a = A(0), b = A(0);
          for (int q = 0; q < kGroups; ++q) {  // fixed order
            a += lds[((q * kE + j) * kL + l) * 2];
            b += lds[((q * kE + j) * kL + l) * 2 + 1];
          }
          out[2 * e] = a;
          out[2 * e + 1] = b;
        }
      }
    }
  }
};

// LayerNorm backward rows that take the staged kernel: as for the forward.
inline bool layer_norm_grad_short_rows(int64_t G, int64_t D, int64_t S, size_t elem_bytes,
                                       const void* x, const void* dy, const void* dx) {
  if (G != 1 || S != 1 || D > 1024 || !congruent16(x, dy) || !congruent16(x, dx)) return false;
  const size_t row_bytes = static_cast<size_t>(D) * elem_bytes;
  return row_bytes <= 512 || row_bytes % 16 != 0 || !aligned16(x);
}
inline unsigned short_grad_grid(int64_t N, uint32_t rows_per_chunk) {
  const unsigned grid = short_grid(N, rows_per_chunk);
  return grid < static_cast<unsigned>(short_grad_max_grid()) ? grid : short_grad_max_grid();
}

// --------------------------------------------------------------------------
// LayerNorm backward of rows wider than the register tiles (flattened feature
// maps, vocabulary-sized rows): two passes over x and dy.
//   1. row sums: a row is cut into `splits` column ranges, one workgroup each,
//      which writes the range's (sum gamma*dy*x, sum gamma*dy) pair;
//   2. a workgroup owns 256*kW adjacent columns of a chunk of rows: a thread
//      keeps gamma, dgamma and dbeta of its kW columns in registers, walks the
//      chunk's rows (adding up the row's pairs in fixed order), writes dx and
//      leaves one partial (dgamma, dbeta) row per chunk for sum_partial_rows.
// kW is a whole packet for rows of aligned packets and 1 otherwise.
// --------------------------------------------------------------------------
constexpr int kWideRowsAhead = 4;  // rows whose loads are in flight per thread

struct WideGradPlan {
  uint32_t col_blocks;      // workgroups across a row in the second pass
  uint32_t row_chunks;      // partial (dgamma, dbeta) rows
  uint32_t rows_per_chunk;
  uint32_t splits;          // workgroups per row in the first pass
  uint32_t split_cols;      // columns per split, whole workgroup tiles
};

inline WideGradPlan plan_wide_grad(int64_t N, int64_t D, int kw) {
  WideGradPlan p;
  const int64_t tile = static_cast<int64_t>(kReduceThreads) * kw;
  const int64_t col_blocks = ceil_div(D, tile);
  // first pass: enough workgroups for the chip, at least four tiles each
  int64_t splits = ceil_div(static_cast<int64_t>(num_cus()) * 4, N);
  const int64_t max_splits = col_blocks / 4 > 1 ? col_blocks / 4 : 1;
  if (splits > max_splits) splits = max_splits;
  const int64_t tiles_per_split = ceil_div(col_blocks, splits);
  splits = ceil_div(col_blocks, tiles_per_split);
  // second pass: about eight workgroups per compute unit, eight rows or more per chunk
  int64_t chunks = ceil_div(static_cast<int64_t>(num_cus()) * 8, col_blocks);
  const int64_t max_chunks = N / 8 > 1 ? N / 8 : 1;
  if (chunks > max_chunks) chunks = max_chunks;
  const int64_t rows_per_chunk = ceil_div(N, chunks);
  chunks = ceil_div(N, rows_per_chunk);
  p.col_blocks = static_cast<uint32_t>(col_blocks);
  p.row_chunks = static_cast<uint32_t>(chunks);
  p.rows_per_chunk = static_cast<uint32_t>(rows_per_chunk);
  p.splits = static_cast<uint32_t>(splits);
  p.split_cols = static_cast<uint32_t>(tiles_per_split * tile);
  return p;
}

// Words of scratch: the row pairs (rounded to whole packets), then the partial rows.
inline size_t wide_grad_pair_words(int64_t N, const WideGradPlan& p) {
  return (static_cast<size_t>(N) * p.splits * 2 + 3) / 4 * 4;
}
inline size_t wide_grad_words(int64_t N, int64_t D, int kw) {
  const WideGradPlan p = plan_wide_grad(N, D, kw);
  return wide_grad_pair_words(N, p) + static_cast<size_t>(p.row_chunks) * D * 2;
}

template <typename T, int kW>
__device__ __forceinline__ void load_run(const T* p, typename IO<T>::Acc (&v)[kW]) {
  if constexpr (kW == 1) {
    v[0] = IO<T>::load1(p);
  } else {
    IO<T>::unpack(load_packet_keep(p), v);
  }
}
template <int kW, typename A>
__device__ __forceinline__ void load_param_run(const A* p, A (&v)[kW]) {
  if constexpr (kW == 1) {
    v[0] = *p;
  } else {
    load_params<kW>(p, v);
  }
}

template <typename T, int kW>
__global__ __launch_bounds__(kReduceThreads) void layer_norm_wide_row_sums(
    const int D, const WideGradPlan p, const T* __restrict__ x, const T* __restrict__ dy,
    const typename IO<T>::Acc* __restrict__ gamma, typename IO<T>::Acc* __restrict__ pairs) {
  using A = typename IO<T>::Acc;
  __shared__ A lds[2 * kReduceWaves];
  const int64_t row = blockIdx.x / p.splits;
  const uint32_t split = blockIdx.x % p.splits;
  const int c0 = static_cast<int>(split * p.split_cols);
  const int c1 = D - c0 < static_cast<int>(p.split_cols) ? D : c0 + static_cast<int>(p.split_cols);
  const T* xr = x + row * D;
  const T* dyr = dy + row * D;
  A s1 = A(0), s2 = A(0);
#pragma unroll 4
  for (int c = c0 + static_cast<int>(threadIdx.x) * kW; c < c1; c += kReduceThreads * kW) {
    A xv[kW], dv[kW], g[kW];
    load_run<T, kW>(xr + c, xv);
    load_run<T, kW>(dyr + c, dv);
    load_param_run<kW>(gamma + c, g);
#pragma unroll
    for (int e = 0; e < kW; ++e) {
      const A t = g[e] * dv[e];
      s1 += t * xv[e];
      s2 += t;
    }
  }
  block_reduce_pair(s1, s2, lds);
  if (threadIdx.x == 0) {
    pairs[static_cast<size_t>(blockIdx.x) * 2] = s1;
    pairs[static_cast<size_t>(blockIdx.x) * 2 + 1] = s2;
  }
}

template <typename T, int kW>
__global__ __launch_bounds__(kReduceThreads) void layer_norm_wide_grad(
    const int64_t N, const int D, const WideGradPlan p, const T* __restrict__ x,
    const T* __restrict__ dy, const typename IO<T>::Acc* __restrict__ gamma,
    const typename IO<T>::Acc* __restrict__ mu, const typename IO<T>::Acc* __restrict__ rsig,
    const typename IO<T>::Acc* __restrict__ pairs, typename IO<T>::Acc* __restrict__ ds,
    typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  const uint32_t block = blockIdx.x % p.col_blocks;  // neighbours share rows
  const uint32_t chunk = blockIdx.x / p.col_blocks;
  const int col = static_cast<int>(block * kReduceThreads + threadIdx.x) * kW;
  const bool active = col < D;
  const int at = active ? col : 0;  // threads past the row address its start and store nothing
  const bool reports = block == 0 && threadIdx.x == 0;
  const A inv_d = A(1) / A(D);
  A g[kW], dg[kW], dbt[kW];
  load_param_run<kW>(gamma + at, g);
#pragma unroll
  for (int e = 0; e < kW; ++e) dg[e] = dbt[e] = A(0);

  const int64_t r0 = static_cast<int64_t>(chunk) * p.rows_per_chunk;
  const int64_t r1 = N - r0 < static_cast<int64_t>(p.rows_per_chunk) ? N : r0 + p.rows_per_chunk;
  for (int64_t r = r0; r < r1; r += kWideRowsAhead) {
    A xv[kWideRowsAhead][kW], dv[kWideRowsAhead][kW];
    A m[kWideRowsAhead], rs[kWideRowsAhead], s1[kWideRowsAhead], s2[kWideRowsAhead];
#pragma unroll
    for (int u = 0; u < kWideRowsAhead; ++u) {
      const int64_t rr = r + u < r1 ? r + u : r1 - 1;  // uniform over the workgroup
      load_run<T, kW>(x + rr * D + at, xv[u]);
      load_run<T, kW>(dy + rr * D + at, dv[u]);
      m[u] = mu[rr];
      rs[u] = rsig[rr];
      s1[u] = s2[u] = A(0);
      const A* pr = pairs + static_cast<size_t>(rr) * p.splits * 2;
      for (uint32_t s = 0; s < p.splits; ++s) {
        s1[u] += pr[2 * s];
        s2[u] += pr[2 * s + 1];
      }
    }
#pragma unroll
    for (int u = 0; u < kWideRowsAhead; ++u) {
      if (r + u < r1) {
        if (reports) {
          ds[r + u] = s1[u];
          db[r + u] = s2[u];
        }
        const A a = (s2[u] * m[u] - s1[u]) * (rs[u] * rs[u] * rs[u]) * inv_d;
        const A b = -(s2[u] * rs[u]) * inv_d;
        if (active) {
#pragma unroll
          for (int e = 0; e < kW; ++e) {
            const A xc = xv[u][e] - m[u];
            const A w = dv[u][e] * rs[u];
            dg[e] += w * xc;
            dbt[e] += dv[u][e];
            xv[u][e] = g[e] * w + (a * xc + b);
          }
          T* out = dx + (r + u) * D + col;
          if constexpr (kW == 1) {
            IO<T>::store1(out, xv[u][0]);
          } else {
            store_packet(out, IO<T>::pack(xv[u]));
          }
        }
      }
    }
  }
  if (active) {
    A* out = partial + (static_cast<size_t>(chunk) * D + col) * 2;
#pragma unroll
    for (int e = 0; e < kW; ++e) {
      out[2 * e] = dg[e];
      out[2 * e + 1] = dbt[e];
    }
  }
}

// --------------------------------------------------------------------------
// Fused group paths (NCHW): a group's D*S elements are contiguous, so a group
// is a row of width L = D*S whose affine parameters change every S elements.
// --------------------------------------------------------------------------

// Moments -> InvStd -> GroupNorm in one pass over x: the group stays in
// registers between the statistics and the normalisation.
// kAnyS: a channel is not whole packets (the group still is), so the elements
// of a packet may belong to different channels; 2 where a channel is 64 packets'
// worth or more, 1 for shorter ones.
template <typename T, int kTPR, int kVPT, int kAnyS = 0>
__global__ __launch_bounds__(row_threads(kTPR)) void group_norm_forward_rows(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = L / kVec;
  const A inv_l = A(1) / A(L);
  const int lane = Tile::lane();

  // The 1024-thread tile (one or two workgroups per compute unit) requests the
  // next group's packets before it reduces the current group.
  constexpr bool kPrefetch = kTPR == 1024;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock;
  int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
  // The loaded packets are not masked (a select on them would wait for each
  // load where it stands): slots beyond the group repeat its first packet and
  // are skipped by the sums and the stores.
  Raw t;
  if (kPrefetch) t.load_unmasked(x + (row < rows ? row : 0) * L, npackets);
  for (; row < rows; row += stride) {
    Raw nxt;
    if (kPrefetch) {
      const bool more = row + stride < rows;
      nxt.load_unmasked(x + (more ? row + stride : 0) * L, npackets);
    } else {
      t.load_unmasked(x + row * L, npackets);
    }
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        A v[kVec];
        t.unpack(i, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) s += v[e];
      }
    }
    const A mean = Tile::reduce(s, SumOp(), slots[0]) * inv_l;
    t.refresh();
    A q = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        A v[kVec];
        t.unpack(i, v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A d = v[e] - mean;
          q += d * d;
        }
      }
    }
    const A var = Tile::reduce(q, SumOp(), slots[1]) * inv_l;
    const A rs = acc_rsqrt_exact(var + eps);
    if (lane == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;
    t.refresh();
    // Results replace the packets in place; they are stored after the wait for
    // the prefetched group so that the stores overlap the next group's work.
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const uint32_t col = static_cast<uint32_t>(i * kTPR + lane) * kVec;
      const uint32_t first = Tile::active(i, npackets) ? col / S : 0u;
      A v[kVec];
      t.unpack(i, v);
      if constexpr (kAnyS == 2) {
        {
          // The wavefront's 64 packets lie in at most two channels, and the
          // boundary in the packet of one lane: its place and both channels'
          // parameters are uniform over the wavefront (scalar registers); only
          // that lane picks per element.
          const uint32_t e0 = static_cast<uint32_t>(
              i * kTPR + __builtin_amdgcn_readfirstlane(lane / kWaveSize) * kWaveSize) * kVec;
          uint32_t chan = e0 / S;
          uint32_t in_first = (chan + 1) * S - e0;
          if (chan >= D) chan = D - 1, in_first = kWaveSize * kVec;
          const uint32_t ca = c0 + chan, cb = c0 + (chan + 1 < D ? chan + 1 : chan);
          const A ga = gamma[ca] * rs, gb = gamma[cb] * rs, ba = beta[ca], bb = beta[cb];
          const int edge = static_cast<int>(in_first / kVec), km = static_cast<int>(in_first % kVec);
          const int wave_lane = lane & (kWaveSize - 1);
          if (km == 0 || wave_lane != edge) {
            const A gam = wave_lane < edge ? ga : gb, bet = wave_lane < edge ? ba : bb;
#pragma unroll
            for (int e = 0; e < kVec; ++e) v[e] = (v[e] - mean) * gam + bet;
          } else {
#pragma unroll
            for (int e = 0; e < kVec; ++e) v[e] = (v[e] - mean) * (e < km ? ga : gb) + (e < km ? ba : bb);
          }
        }
      } else if constexpr (kAnyS == 1) {
        const uint32_t rem = Tile::active(i, npackets) ? col - first * S : 0u;
        if (S >= static_cast<uint32_t>(kVec)) {
          // at most two channels per packet: their parameters once, picked per element
          const uint32_t ca = c0 + first, cb = c0 + (first + 1 < D ? first + 1 : first);
          const A ga = gamma[ca] * rs, gb = gamma[cb] * rs, ba = beta[ca], bb = beta[cb];
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            const bool second = rem + e >= S;
            v[e] = (v[e] - mean) * (second ? gb : ga) + (second ? bb : ba);
          }
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            uint32_t k = rem + e, c = first;
            while (k >= S) k -= S, ++c;
            c = c0 + (c < D ? c : D - 1);
            v[e] = (v[e] - mean) * (gamma[c] * rs) + beta[c];
          }
        }
      } else {
        const uint32_t c = c0 + first;  // kVec divides S
        const A gam = gamma[c] * rs, bet = beta[c];
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = (v[e] - mean) * gam + bet;
      }
      t.p[i] = IO<T>::pack(v);
    }
    if (kPrefetch) nxt.wait_ready();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        store_packet(y + row * L + static_cast<int64_t>(i * kTPR + lane) * kVec, t.p[i]);
      }
    }
    if (kTPR != kWaveSize) __syncthreads();
    if (kPrefetch) t = nxt;
  }
}

// The same for groups that are not whole aligned packets (D * S odd, or a base
// that is not 16-byte aligned), x and y congruent modulo 16 bytes: a group is
// read as the aligned packets that cover it (RowWindow; the tile is sized for
// L / kVec + 2 packets) and kept as raw packets. A packet wholly inside the
// group that lies in one channel takes the packet code; the packets at the
// group's ends and those across two channels go element by element; the
// elements of the neighbouring groups in the two end packets are neither summed
// nor stored.
template <typename T, int kTPR, int kVPT>
__global__ __launch_bounds__(row_threads(kTPR)) void group_norm_forward_rows_windows(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const A inv_l = A(1) / A(L);
  const int lane = Tile::lane();
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < rows; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    const T* xr = x + row * L;
    const RowWindow<T> w(xr, L);
    const int npackets = w.packets;
    Raw t;
    t.load_unmasked(xr - w.lead, npackets);
    // slot i of this lane: its first element's place in the group (below zero in the
    // group's first packet), and whether all of its elements belong to the group
    auto col_of = [&](int i) { return (i * kTPR + lane) * kVec - w.lead; };
    auto whole = [&](int col) { return col >= 0 && col + kVec <= L; };
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        const int col = col_of(i);
        A v[kVec];
        t.unpack(i, v);
        if (whole(col)) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) s += v[e];
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) s += col + e >= 0 && col + e < L ? v[e] : A(0);
        }
      }
    }
    const A mean = Tile::reduce(s, SumOp(), slots[0]) * inv_l;
    t.refresh();
    A q = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        const int col = col_of(i);
        A v[kVec];
        t.unpack(i, v);
        const bool all = whole(col);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A d = v[e] - mean;
          q += all || (col + e >= 0 && col + e < L) ? d * d : A(0);
        }
      }
    }
    const A var = Tile::reduce(q, SumOp(), slots[1]) * inv_l;
    const A rs = acc_rsqrt_exact(var + eps);
    if (lane == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;
    T* yr = y + row * L;
    t.refresh();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        const int col = col_of(i);
        const uint32_t colp = static_cast<uint32_t>(col < 0 ? 0 : col);
        const uint32_t first = colp / S;
        const uint32_t rem = colp - first * S;
        A v[kVec];
        t.unpack(i, v);
        if (col >= 0 && rem + kVec <= S) {  // the packet lies within one channel
          const A gam = gamma[c0 + first] * rs, bet = beta[c0 + first];
#pragma unroll
          for (int e = 0; e < kVec; ++e) v[e] = (v[e] - mean) * gam + bet;
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            int k = static_cast<int>(rem) + e + (col < 0 ? col : 0);
            if (k < 0) k = 0;  // before the group: not stored
            uint32_t c = first;
            while (static_cast<uint32_t>(k) >= S) k -= static_cast<int>(S), ++c;
            if (c >= D) c = D - 1;  // beyond the group: not stored
            v[e] = (v[e] - mean) * (gamma[c0 + c] * rs) + beta[c0 + c];
          }
        }
        if (whole(col)) {
          store_packet(yr + col, IO<T>::pack(v));
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (col + e >= 0 && col + e < L) IO<T>::store1(yr + col + e, v[e]);
          }
        }
      }
    }
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// The same for any S and any alignment (S not a multiple of a packet, so
// that a packet may straddle channels and groups start at element-aligned
// addresses): ragged tiles, the channel of an element found from its column.
// (x and y not congruent modulo 16 bytes; congruent tensors take the windows above.)
template <typename T, int kTPR, int kVPT>
__global__ __launch_bounds__(row_threads(kTPR)) void group_norm_forward_rows_any(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), true>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const A inv_l = A(1) / A(L);
  const int lane = Tile::lane();
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < rows; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    constexpr int lead = 0;
    const int extent = L;
    Tile t;
    t.load(x + row * L, L, A(0));
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += t.v[i][e];
    const A mean = Tile::reduce(s, SumOp(), slots[0]) * inv_l;
    A q = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const A d = t.v[i][e] - mean;
        const int col = (i * kTPR + lane) * kVec + e - lead;
        if (col >= 0 && col < L) q += d * d;
      }
    const A var = Tile::reduce(q, SumOp(), slots[1]) * inv_l;
    const A rs = acc_rsqrt_exact(var + eps);
    if (lane == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, extent)) {
        const int col = (i * kTPR + lane) * kVec - lead;  // below zero: the group's first packet
        const uint32_t colp = static_cast<uint32_t>(col < 0 ? 0 : col);
        const uint32_t first = colp / S;
        const uint32_t rem = colp - first * S;
        if (col >= 0 && rem + kVec <= S) {  // the packet lies within one channel
          const A gam = gamma[c0 + first] * rs, bet = beta[c0 + first];
#pragma unroll
          for (int e = 0; e < kVec; ++e) t.v[i][e] = (t.v[i][e] - mean) * gam + bet;
        } else {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            int k = static_cast<int>(rem) + e + (col < 0 ? col : 0);
            if (k < 0) k = 0;  // before the group: not stored
            uint32_t c = first;
            while (static_cast<uint32_t>(k) >= S) k -= static_cast<int>(S), ++c;
            if (c >= D) c = D - 1;  // padding beyond the group: not stored
            t.v[i][e] = (t.v[i][e] - mean) * (gamma[c0 + c] * rs) + beta[c0 + c];
          }
        }
      }
    }
    t.store(y + row * L, L);
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// GroupNormGrad in one pass over x and dy: one workgroup per group keeps both
// as raw packets. A (slot, wavefront) pair covers 64 adjacent packets of the
// group. Where S is a multiple of 64 packets these lie in one channel, and the
// per-channel sums are a wave reduction plus a fixed-order sum over LDS
// entries (kChannelWaves). kChannelStraddles takes any S of at least 64 whole
// packets: the 64 packets then lie in at most two channels, split at a lane
// known per wavefront, so gamma is one of two scalars and a pair contributes a
// sum to each of them. kChannelLanes takes channels of 1, 2, 4 .. 32 packets:
// a channel is a group of adjacent lanes of one (slot, wavefront) pair, reduced
// with shuffles and written by its first lane; gamma is read per lane.
// partial[(n*C + c)*2 + {0,1}] receives this group's share of dgamma / dbeta.
// kChannelStraddlesAny is kChannelStraddles for channels that are not whole
// packets (S any number of elements from 64 packets' worth on, the group still
// whole aligned packets): the 64 packets of a (slot, wavefront) pair lie in at
// most two channels, and the boundary may fall inside one packet, whose lane
// then picks gamma and the channel share per element.
enum ChannelMode {
  kChannelWaves = 0,
  kChannelStraddles = 1,
  kChannelLanes = 2,
  kChannelPackets = 3,
  kChannelStraddlesAny = 4
};
// kChannelPackets (group_norm_grad_rows_any): at most this many packets per
// group, 4 accumulator words of LDS each.
constexpr int kMaxEntryPackets = 4096;

template <typename T, int kTPR, int kVPT, int kMode>
__global__ __launch_bounds__(kTPR, kTPR == 512 ? 4 : 1) void group_norm_grad_rows(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const T* __restrict__ x, const T* __restrict__ dy,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ mu,
    const typename IO<T>::Acc* __restrict__ rsig, typename IO<T>::Acc* __restrict__ ds,
    typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial) {
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  constexpr int kWaves = kTPR / kWaveSize;
  constexpr bool kAnyS = kMode == kChannelStraddlesAny;
  constexpr bool kStraddle = kMode == kChannelStraddles || kAnyS;
  constexpr bool kLanes = kMode == kChannelLanes;
  // kChannelWaves: the 64 packets of a (slot, wavefront) pair lie in one channel, so their
  // sums of dy * x and dy, reduced over the wavefront in the first pass, give the group's ds /
  // db shares (times gamma, a scalar) and the channel's dgamma / dbeta shares
  // ((sum(dy x) - mu sum(dy)) rsig, as the CPU kernel forms them per (n, c)) at once; the second
  // pass is then two multiply-adds per element and reduces nothing.
  constexpr bool kWholeWaves = kMode == kChannelWaves;
  constexpr int kParts = kStraddle ? 4 : 2;  // per entry: (dgamma, dbeta) of one or two channels
  __shared__ A slots[2 * Tile::kSlots];
  __shared__ A chan_part[kVPT][kWaves][kParts];
  const int npackets = L / kVec;
  const uint32_t packets_per_chan = S / kVec;
  const A denom = A(1) / A(L);
  const int lane = threadIdx.x;
  const int wave_lane = lane & (kWaveSize - 1);
  // Uniform over the wavefront, so everything indexed by it (the channel of a
  // slot, its gamma) stays in scalar registers.
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / kWaveSize));

  // The first channel of the 64 packets of (slot i, this wavefront), and how
  // many of them lie in it (64 or more: all). Packets beyond the group take
  // the last channel.
  auto first_channel = [&](int i, uint32_t& chan, uint32_t& in_first) {
    const uint32_t p0 = static_cast<uint32_t>(i * kTPR + wave * kWaveSize);
    chan = p0 / packets_per_chan;
    in_first = (chan + 1) * packets_per_chan - p0;
    if (chan >= D) chan = D - 1, in_first = kWaveSize;
  };
  // kAnyS, the same in elements: the channel of the first element of the 64
  // packets, and how many of their 64 * kVec elements lie in it.
  constexpr uint32_t kSpan = kWaveSize * kVec;
  auto first_channel_elems = [&](int i, uint32_t& chan, uint32_t& in_first) {
    // (16-bit types: found again at every use. Kept per slot across the passes, the
    // boundaries and both gammas spill 156 bytes at eight packets per thread and
    // tensor; fp32 has the registers and is 5-9% faster keeping them.)
    int w = wave;
    if constexpr (sizeof(T) == 2) asm volatile("" : "+s"(w));
    const uint32_t e0 = static_cast<uint32_t>(i * kTPR + w * kWaveSize) * kVec;
    chan = e0 / S;
    in_first = (chan + 1) * S - e0;
    if (chan >= D) chan = D - 1, in_first = kSpan;
  };

  // A workgroup fills the compute unit's registers, so the next group cannot be
  // held beside the current one: its packets are requested slot by slot into the
  // registers the second pass has just finished with, and are in flight while
  // the rest of this group is computed, stored and reduced.
  // The loaded packets are not masked: packets beyond the group skip the sums.
  Raw tx, tdy;
  if (blockIdx.x < rows) {
    tx.load_unmasked(x + static_cast<int64_t>(blockIdx.x) * L, npackets);
    tdy.load_unmasked(dy + static_cast<int64_t>(blockIdx.x) * L, npackets);
  }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int64_t next = row + gridDim.x;
    const bool next_valid = next < rows;
    const T* nx = x + (next_valid ? next : row) * L;
    const T* ndy = dy + (next_valid ? next : row) * L;
    const A m = mu[row], r = rsig[row];
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;

    A gam[kVPT];
    A s1 = A(0), s2 = A(0);
    if constexpr (kLanes) {
      // A channel is packets_per_chan (a power of two below 64) adjacent lanes of a slot. The
      // slots' sums of dy x and dy are added up over them with xor-shuffles, four slots' worth
      // in flight together (one slot after the other, between the stores of the second pass,
      // each shuffle waited for the one before it), and the channel's first lane writes its
      // (dgamma, dbeta) share, (sum(dy x) - mu sum(dy)) rsig as the CPU kernel forms it per (n, c).
      constexpr int kBatch = kVPT >= 4 ? 4 : kVPT;
      const size_t n = static_cast<size_t>(row / G);
#pragma unroll
      for (int b = 0; b < kVPT; b += kBatch) {
        A chan1[kBatch], chan2[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          const int i = b + j;
          const uint32_t chan = static_cast<uint32_t>(i * kTPR + lane) / packets_per_chan;
          gam[i] = gamma[c0 + (chan < D ? chan : D - 1)];
          A p1 = A(0), p2 = A(0);
          if (Tile::active(i, npackets)) {
            A xv[kVec], dv[kVec];
            tx.unpack(i, xv);
            tdy.unpack(i, dv);
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              p1 += dv[e] * xv[e];
              p2 += dv[e];
            }
          }
          s1 += gam[i] * p1;
          s2 += gam[i] * p2;
          chan1[j] = p1, chan2[j] = p2;
        }
        for (uint32_t o = 1; o < packets_per_chan; o <<= 1) {
#pragma unroll
          for (int j = 0; j < kBatch; ++j) {
            chan1[j] += __shfl_xor(chan1[j], static_cast<int>(o), kWaveSize);
            chan2[j] += __shfl_xor(chan2[j], static_cast<int>(o), kWaveSize);
          }
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          const int i = b + j;
          const uint32_t packet = static_cast<uint32_t>(i * kTPR + lane);
          if ((packet & (packets_per_chan - 1)) == 0 && Tile::active(i, npackets)) {
            A* o = partial + (n * G * D + c0 + packet / packets_per_chan) * 2;
            o[0] = (chan1[j] - m * chan2[j]) * r;
            o[1] = chan2[j];
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < (kLanes ? 0 : kVPT); ++i) {
      if constexpr (kAnyS) {
        uint32_t chan, in_first;
        first_channel_elems(i, chan, in_first);
        const A ga = gamma[c0 + chan], gb = gamma[c0 + (chan + 1 < D ? chan + 1 : chan)];
        // The boundary falls into the packet of lane `edge`, `km` elements into
        // it (0: between two packets); both are uniform over the wavefront.
        const int edge = static_cast<int>(in_first / kVec), km = static_cast<int>(in_first % kVec);
        if (Tile::active(i, npackets)) {
          A xv[kVec], dv[kVec];
          tx.unpack(i, xv);
          tdy.unpack(i, dv);
          if (km == 0 || wave_lane != edge) {
            A p1 = A(0), p2 = A(0);
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              p1 += dv[e] * xv[e];
              p2 += dv[e];
            }
            const A g = wave_lane < edge ? ga : gb;
            s1 += g * p1;
            s2 += g * p2;
          } else {
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              const A t = (e < km ? ga : gb) * dv[e];
              s1 += t * xv[e];
              s2 += t;
            }
          }
        }
      } else if constexpr (kLanes) {
        // (handled above)
      } else if constexpr (kWholeWaves) {
        uint32_t chan, in_first;
        first_channel(i, chan, in_first);
        gam[i] = gamma[c0 + chan];
        A p1 = A(0), p2 = A(0);
        if (Tile::active(i, npackets)) {
          A xv[kVec], dv[kVec];
          tx.unpack(i, xv);
          tdy.unpack(i, dv);
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            p1 += dv[e] * xv[e];
            p2 += dv[e];
          }
        }
        p1 = wave_allreduce(p1, SumOp());
        p2 = wave_allreduce(p2, SumOp());
        if (wave_lane == 0) {
          chan_part[i][wave][0] = (p1 - m * p2) * r;
          chan_part[i][wave][1] = p2;
        }
        s1 += gam[i] * p1;  // (the same in every lane: the wavefront's share)
        s2 += gam[i] * p2;
      } else {
        uint32_t chan, in_first;
        first_channel(i, chan, in_first);
        gam[i] = gamma[c0 + chan];
        if constexpr (kStraddle) {
          const A second = gamma[c0 + (chan + 1 < D ? chan + 1 : chan)];
          gam[i] = static_cast<uint32_t>(wave_lane) < in_first ? gam[i] : second;
        }
      }
      if (!kAnyS && !kWholeWaves && !kLanes && Tile::active(i, npackets)) {
        // gamma is one value per thread and slot: it multiplies the slot's sums once
        A xv[kVec], dv[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        A p1 = A(0), p2 = A(0);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          p1 += dv[e] * xv[e];
          p2 += dv[e];
        }
        s1 += gam[i] * p1;
        s2 += gam[i] * p2;
      }
    }
    if constexpr (kWholeWaves) {
      if (wave_lane == 0) slots[2 * wave] = s1, slots[2 * wave + 1] = s2;
      __syncthreads();
      s1 = s2 = A(0);
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        s1 += slots[2 * w];
        s2 += slots[2 * w + 1];
      }
    } else {
      Tile::reduce_sum_pair(s1, s2, slots);
    }
    if (lane == 0) {
      ds[row] = s1;
      db[row] = s2;
    }
    // dx = gamma*rsig * dy + (u*(x - mu) - v) with the row's u, v divided by D*S once
    const A u0 = (s2 * m - s1) * (r * r * r) * denom;
    const A v0 = s2 * r * denom;
    const A w0 = -(u0 * m + v0);  // kWholeWaves, kLanes: dx = gamma*rsig * dy + (u x + w)
    tx.refresh();
    tdy.refresh();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      A t1 = A(0), t2 = A(0);
      A u1 = A(0), u2 = A(0);  // kAnyS: the second channel's share of a packet on the boundary
      if constexpr (kWholeWaves || kLanes) {
        if (Tile::active(i, npackets)) {
          A xv[kVec], dv[kVec];
          tx.unpack(i, xv);
          tdy.unpack(i, dv);
          const A gr = gam[i] * r;
#pragma unroll
          for (int e = 0; e < kVec; ++e) xv[e] = gr * dv[e] + (u0 * xv[e] + w0);
          tx.store_slot(dx + row * L, i, xv);
        }
      } else if constexpr (kAnyS) {
        uint32_t chan, in_first;
        first_channel_elems(i, chan, in_first);
        const int edge = static_cast<int>(in_first / kVec), km = static_cast<int>(in_first % kVec);
        if (Tile::active(i, npackets)) {
          const A ga = gamma[c0 + chan] * r, gb = gamma[c0 + (chan + 1 < D ? chan + 1 : chan)] * r;
          A xv[kVec], dv[kVec];
          tx.unpack(i, xv);
          tdy.unpack(i, dv);
          if (km == 0 || wave_lane != edge) {
            const A gr = wave_lane < edge ? ga : gb;
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              const A xc = xv[e] - m;
              t1 += dv[e] * xc;
              t2 += dv[e];
              xv[e] = gr * dv[e] + (u0 * xc - v0);
            }
            if (wave_lane >= edge) u1 = t1, u2 = t2, t1 = A(0), t2 = A(0);
          } else {
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              const bool head = e < km;
              const A xc = xv[e] - m;
              const A w = dv[e] * xc;
              t1 += head ? w : A(0);
              t2 += head ? dv[e] : A(0);
              u1 += head ? A(0) : w;
              u2 += head ? A(0) : dv[e];
              xv[e] = (head ? ga : gb) * dv[e] + (u0 * xc - v0);
            }
          }
          t1 *= r;
          u1 *= r;
          tx.store_slot(dx + row * L, i, xv);
        }
      } else if (Tile::active(i, npackets)) {
        A xv[kVec], dv[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        const A gr = gam[i] * r;
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A xc = xv[e] - m;
          t1 += dv[e] * xc;
          t2 += dv[e];
          xv[e] = gr * dv[e] + (u0 * xc - v0);
        }
        t1 *= r;
        tx.store_slot(dx + row * L, i, xv);
      }
      if (next_valid) {
        tx.load_slot_unmasked(nx, i, npackets);
        tdy.load_slot_unmasked(ndy, i, npackets);
      }
      if constexpr (kAnyS) {
        uint32_t chan, in_first;
        first_channel_elems(i, chan, in_first);
        const A a1 = wave_allreduce(t1, SumOp());
        const A a2 = wave_allreduce(t2, SumOp());
        A b1 = A(0), b2 = A(0);
        if (in_first < kSpan) {  // uniform over the wavefront
          b1 = wave_allreduce(u1, SumOp());
          b2 = wave_allreduce(u2, SumOp());
        }
        if (wave_lane == 0) {
          chan_part[i][wave][0] = a1;
          chan_part[i][wave][1] = a2;
          chan_part[i][wave][2] = b1;
          chan_part[i][wave][3] = b2;
        }
      } else if constexpr (kLanes) {
        // (its channel sums left the first pass)
      } else if constexpr (kStraddle) {
        uint32_t chan, in_first;
        first_channel(i, chan, in_first);
        const bool head = static_cast<uint32_t>(wave_lane) < in_first;
        const A a1 = wave_allreduce(head ? t1 : A(0), SumOp());
        const A a2 = wave_allreduce(head ? t2 : A(0), SumOp());
        A b1 = A(0), b2 = A(0);
        if (in_first < static_cast<uint32_t>(kWaveSize)) {  // uniform over the wavefront
          b1 = wave_allreduce(head ? A(0) : t1, SumOp());
          b2 = wave_allreduce(head ? A(0) : t2, SumOp());
        }
        if (wave_lane == 0) {
          chan_part[i][wave][0] = a1;
          chan_part[i][wave][1] = a2;
          chan_part[i][wave][2] = b1;
          chan_part[i][wave][3] = b2;
        }
      } else if constexpr (!kWholeWaves) {
        t1 = wave_allreduce(t1, SumOp());
        t2 = wave_allreduce(t2, SumOp());
        if (wave_lane == 0) {
          chan_part[i][wave][0] = t1;
          chan_part[i][wave][1] = t2;
        }
      }
    }
    __syncthreads();
    if (!kLanes && static_cast<uint32_t>(lane) < D) {
      // Entry q = (slot, wavefront) covers packets [64 q, 64 q + 64); channel
      // `lane` owns the packets [lane * packets_per_chan, (lane + 1) * packets_per_chan).
      A a = A(0), b = A(0);
      const A* entries = &chan_part[0][0][0];
      if constexpr (kAnyS) {
        // the same in elements: entry q covers elements [q kSpan, (q + 1) kSpan)
        const uint32_t lo = static_cast<uint32_t>(lane) * S;
        const uint32_t q0 = lo / kSpan, q1 = (lo + S - 1) / kSpan;
#pragma nounroll
        for (uint32_t q = q0; q <= q1; ++q) {
          const uint32_t part = q * kSpan >= lo ? 0u : 2u;
          a += entries[4 * q + part];
          b += entries[4 * q + part + 1];
        }
      } else if constexpr (kStraddle) {
        const uint32_t lo = static_cast<uint32_t>(lane) * packets_per_chan;
        const uint32_t q0 = lo / kWaveSize, q1 = (lo + packets_per_chan - 1) / kWaveSize;
#pragma nounroll
        for (uint32_t q = q0; q <= q1; ++q) {
          // the entry's first packet lies in this channel or in the one before it
          const uint32_t part = q * kWaveSize >= lo ? 0u : 2u;
          a += entries[4 * q + part];
          b += entries[4 * q + part + 1];
        }
      } else {
        const uint32_t waves_per_chan = packets_per_chan / kWaveSize;
        const uint32_t q0 = static_cast<uint32_t>(lane) * waves_per_chan;
#pragma nounroll
        for (uint32_t q = q0; q < q0 + waves_per_chan; ++q) {
          a += entries[2 * q];
          b += entries[2 * q + 1];
        }
      }
      const size_t n = static_cast<size_t>(row / G);
      A* o = partial + (n * G * D + c0 + lane) * 2;
      o[0] = a;
      o[1] = b;
    }
    __syncthreads();  // chan_part and slots are reused by the next group
  }
}

// The same for groups of whole aligned packets whose channels are not (S is
// not a multiple of a packet but at least one: 14x14 and 7x7 maps): a packet
// holds elements of at most two channels. gamma is one of two values per
// packet, picked per element; a thread leaves the (dgamma, dbeta) shares of
// its packet's first and second channel in LDS, one entry per packet, and the
// thread that owns a channel adds the entries of that channel's packets in
// order. Dynamic LDS: 4 accumulator words per packet of the group.
// kWindow: the groups themselves are not whole aligned packets (D * S odd, or
// bases that are not 16-byte aligned; x, dy and dx congruent modulo 16 bytes).
// A group is read as the aligned packets that cover it; what its two end
// packets hold of the neighbouring groups is replaced by values that add
// nothing to any sum (dy = 0, x = mean) and is not stored. Dynamic LDS then
// holds L / kVec + 2 entries.
template <typename T, int kTPR, int kVPT, bool kWindow = false>
__global__ __launch_bounds__(kTPR) void group_norm_grad_rows_any(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const T* __restrict__ x, const T* __restrict__ dy,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ mu,
    const typename IO<T>::Acc* __restrict__ rsig, typename IO<T>::Acc* __restrict__ ds,
    typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial) {
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2 * Tile::kSlots];
  extern __shared__ u32x4 dynamic_lds[];
  A* entries = reinterpret_cast<A*>(dynamic_lds);  // [npackets][4]
  const A denom = A(1) / A(L);
  const int lane = threadIdx.x;
  // a group's window: elements of its first packet before it, and its packets
  auto lead_of = [&](int64_t row) {
    return kWindow ? RowWindow<T>(x + row * L, L).lead : 0;
  };
  auto packets_of = [&](int lead) { return kWindow ? (lead + L + kVec - 1) / kVec : L / kVec; };

  Raw tx, tdy;
  if (blockIdx.x < rows) {
    const int lead0 = lead_of(blockIdx.x);
    tx.load_unmasked(x + static_cast<int64_t>(blockIdx.x) * L - lead0, packets_of(lead0));
    tdy.load_unmasked(dy + static_cast<int64_t>(blockIdx.x) * L - lead0, packets_of(lead0));
  }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int lead = lead_of(row);
    const int npackets = packets_of(lead);
    const int64_t next = row + gridDim.x;
    const bool next_valid = next < rows;
    const int nlead = lead_of(next_valid ? next : row);
    const int next_packets = packets_of(nlead);
    const T* nx = x + (next_valid ? next : row) * L - nlead;
    const T* ndy = dy + (next_valid ? next : row) * L - nlead;
    const A m = mu[row], r = rsig[row];
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;
    // kWindow: the elements of slot i's packet that belong to the group are [lo, hi)
    auto neutralize = [&](int i, A (&xv)[kVec], A (&dv)[kVec]) {
      if constexpr (kWindow) {
        const int col = (i * kTPR + lane) * kVec - lead;
        if (col < 0 || col + kVec > L) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (col + e < 0 || col + e >= L) xv[e] = m, dv[e] = A(0);
          }
        }
      }
    };

    // Of slot i's packet: the position of its first element in that element's
    // channel, and gamma of that channel and of the next. Found again in the
    // second pass rather than kept: four more registers per slot cost occupancy.
    auto channels_of = [&](int i, uint32_t& rem, A& g0, A& g1) {
      // (kWindow: the group's first packet starts `lead` elements before it; its
      // elements count from the group's first, the ones before it as channel 0)
      const int at = Tile::active(i, npackets) ? (i * kTPR + lane) * kVec - lead : 0;
      const uint32_t col = static_cast<uint32_t>(at < 0 ? 0 : at);
      const uint32_t first = col / S;
      rem = col - first * S;
      g0 = gamma[c0 + first];
      g1 = gamma[c0 + (first + 1 < D ? first + 1 : first)];
    };
    A s1 = A(0), s2 = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        uint32_t rem;
        A g0, g1;
        channels_of(i, rem, g0, g1);
        A xv[kVec], dv[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        neutralize(i, xv, dv);
        const int shift = kWindow && i == 0 && lane == 0 ? lead : 0;  // the first packet's offset
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A t = (rem + e >= S + shift ? g1 : g0) * dv[e];
          s1 += t * xv[e];
          s2 += t;
        }
      }
    }
    Tile::reduce_sum_pair(s1, s2, slots);
    if (lane == 0) {
      ds[row] = s1;
      db[row] = s2;
    }
    const A u0 = (s2 * m - s1) * (r * r * r);
    const A v0 = s2 * r;
    tx.refresh();
    tdy.refresh();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        uint32_t rem;
        A g0, g1;
        channels_of(i, rem, g0, g1);
        A xv[kVec], dv[kVec];
        tx.unpack(i, xv);
        tdy.unpack(i, dv);
        neutralize(i, xv, dv);
        const int shift = kWindow && i == 0 && lane == 0 ? lead : 0;
        A h1 = A(0), h2 = A(0), t1 = A(0), t2 = A(0);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const bool second = rem + e >= S + shift;
          const A xc = xv[e] - m;
          const A w = dv[e] * xc * r;
          h1 += second ? A(0) : w;
          h2 += second ? A(0) : dv[e];
          t1 += second ? w : A(0);
          t2 += second ? dv[e] : A(0);
          xv[e] = (second ? g1 : g0) * dv[e] * r + (u0 * xc - v0) * denom;
        }
        if constexpr (kWindow) {
          const int col = (i * kTPR + lane) * kVec - lead;
          if (col >= 0 && col + kVec <= L) {
            store_packet(dx + row * L + col, IO<T>::pack(xv));
          } else {
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              if (col + e >= 0 && col + e < L) IO<T>::store1(dx + row * L + col + e, xv[e]);
            }
          }
        } else {
          tx.store_slot(dx + row * L, i, xv);
        }
        A* entry = entries + static_cast<size_t>(i * kTPR + lane) * 4;
        entry[0] = h1, entry[1] = h2, entry[2] = t1, entry[3] = t2;
      }
      if (next_valid) {
        tx.load_slot_unmasked(nx, i, next_packets);
        tdy.load_slot_unmasked(ndy, i, next_packets);
      }
    }
    __syncthreads();
    // Channel c owns elements [c S, (c + 1) S), that is the first-channel share
    // of the packets that start in it and the second-channel share of the one
    // that starts before it and reaches in: a thread per channel where a channel
    // is a few dozen packets, a wavefront per channel where it is more.
    const size_t n = static_cast<size_t>(row / G);
    if (S / kVec <= 32) {
      for (uint32_t c = lane; c < D; c += kTPR) {
        // (kWindow: packet p starts at element p * kVec - lead of the group; the
        // first packet's elements before the group count as channel 0)
        const uint32_t lo = c * S + (c == 0 ? 0u : static_cast<uint32_t>(lead));
        const uint32_t p0 = lo / kVec, p1 = (c * S + lead + S - 1) / kVec;
        A a = A(0), b = A(0);
#pragma nounroll
        for (uint32_t p = p0; p <= p1; ++p) {
          const uint32_t part = p * kVec >= lo ? 0u : 2u;
          a += entries[4 * p + part];
          b += entries[4 * p + part + 1];
        }
        A* o = partial + (n * G * D + c0 + c) * 2;
        o[0] = a;
        o[1] = b;
      }
    } else {
      constexpr int kWaves = kTPR / kWaveSize;
      const uint32_t wave = static_cast<uint32_t>(lane) / kWaveSize;
      const uint32_t wave_lane = static_cast<uint32_t>(lane) & (kWaveSize - 1);
      for (uint32_t c = wave; c < D; c += kWaves) {
        // (kWindow: packet p starts at element p * kVec - lead of the group; the
        // first packet's elements before the group count as channel 0)
        const uint32_t lo = c * S + (c == 0 ? 0u : static_cast<uint32_t>(lead));
        const uint32_t p0 = lo / kVec, p1 = (c * S + lead + S - 1) / kVec;
        A a = A(0), b = A(0);
        for (uint32_t p = p0 + wave_lane; p <= p1; p += kWaveSize) {
          const uint32_t part = p * kVec >= lo ? 0u : 2u;
          a += entries[4 * p + part];
          b += entries[4 * p + part + 1];
        }
        a = wave_allreduce(a, SumOp());
        b = wave_allreduce(b, SumOp());
        if (wave_lane == 0) {
          A* o = partial + (n * G * D + c0 + c) * 2;
          o[0] = a;
          o[1] = b;
        }
      }
    }
    __syncthreads();  // entries and slots are reused by the next group
  }
}

// Small groups (up to 256 packets: 14x14 and 7x7 maps with a few channels per
// group), a wavefront per group and four groups per workgroup: nothing is
// shared between the wavefronts, so there is no workgroup barrier. x and dy
// of a group stay in registers; ds / db are wave reductions; a packet holds
// elements of at most two channels (S >= kVec), whose (dgamma, dbeta) shares go
// to one LDS entry per packet in the wavefront's own region, and lane d adds
// the entries of channel d in packet order. partial[(n*C + c)*2 + {0,1}]
// receives this group's share of dgamma / dbeta, as in the kernels above.
constexpr int kWaveGroupThreads = 256;
template <typename T, int kVPT>
__global__ __launch_bounds__(kWaveGroupThreads) void group_norm_grad_wave_groups(
    const int64_t rows, const int L, const uint32_t G, const uint32_t D, const uint32_t S,
    const T* __restrict__ x, const T* __restrict__ dy,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ mu,
    const typename IO<T>::Acc* __restrict__ rsig, typename IO<T>::Acc* __restrict__ ds,
    typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kWaves = kWaveGroupThreads / kWaveSize;
  __shared__ A entries[kWaves][kWaveSize * kVPT][4];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / kWaveSize));
  const int npackets = L / kVec;
  const A denom = A(1) / A(L);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave; row < rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    const T* xr = x + row * L;
    const T* dr = dy + row * L;
    u32x4 rx[kVPT], rd[kVPT];
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int p = i * kWaveSize + lane;
      const int64_t off = static_cast<int64_t>(p < npackets ? p : 0) * kVec;
      rx[i] = load_packet(xr + off);
      rd[i] = load_packet(dr + off);
    }
    const A m = mu[row], r = rsig[row];
    const uint32_t c0 = static_cast<uint32_t>(row % G) * D;
    // of packet p: the position of its first element in that element's channel,
    // and gamma of that channel and of the next
    auto channels_of = [&](int p, uint32_t& rem, A& g0, A& g1) {
      const uint32_t col = static_cast<uint32_t>(p) * kVec;
      const uint32_t first = col / S;
      rem = col - first * S;
      g0 = gamma[c0 + first];
      g1 = gamma[c0 + (first + 1 < D ? first + 1 : first)];
    };
    A s1 = A(0), s2 = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int p = i * kWaveSize + lane;
      if (p < npackets) {
        uint32_t rem;
        A g0, g1;
        channels_of(p, rem, g0, g1);
        A xv[kVec], dv[kVec];
        IO<T>::unpack(rx[i], xv);
        IO<T>::unpack(rd[i], dv);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A t = (rem + e >= S ? g1 : g0) * dv[e];
          s1 += t * xv[e];
          s2 += t;
        }
      }
    }
    s1 = wave_allreduce(s1, SumOp());
    s2 = wave_allreduce(s2, SumOp());
    if (lane == 0) {
      ds[row] = s1;
      db[row] = s2;
    }
    const A u0 = (s2 * m - s1) * (r * r * r);
    const A v0 = s2 * r;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(rx[i]), "+v"(rd[i]));
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int p = i * kWaveSize + lane;
      if (p < npackets) {
        uint32_t rem;
        A g0, g1;
        channels_of(p, rem, g0, g1);
        A xv[kVec], dv[kVec];
        IO<T>::unpack(rx[i], xv);
        IO<T>::unpack(rd[i], dv);
        A h1 = A(0), h2 = A(0), t1 = A(0), t2 = A(0);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const bool second = rem + e >= S;
          const A xc = xv[e] - m;
          const A w = dv[e] * xc * r;
          h1 += second ? A(0) : w;
          h2 += second ? A(0) : dv[e];
          t1 += second ? w : A(0);
          t2 += second ? dv[e] : A(0);
          xv[e] = (second ? g1 : g0) * dv[e] * r + (u0 * xc - v0) * denom;
        }
        store_packet(dx + row * L + static_cast<int64_t>(p) * kVec, IO<T>::pack(xv));
        A* entry = entries[wave][p];
        entry[0] = h1, entry[1] = h2, entry[2] = t1, entry[3] = t2;
      }
    }
    // the wavefront's own entries: its LDS writes are complete before its reads
    __threadfence_block();
    // A channel's entries are shared out among `lanes_per_chan` adjacent lanes (a
    // power of two, so that 64 / lanes_per_chan channels are in work at once), each
    // of which adds every lanes_per_chan-th packet; xor shuffles combine them.
    const size_t n = static_cast<size_t>(row / G);
    uint32_t lanes_per_chan = 1;
    while (lanes_per_chan * 2 * D <= static_cast<uint32_t>(kWaveSize)) lanes_per_chan <<= 1;
    const uint32_t chans_at_a_time = kWaveSize / lanes_per_chan;
    const uint32_t sub = static_cast<uint32_t>(lane) % lanes_per_chan;
    for (uint32_t cb = 0; cb < D; cb += chans_at_a_time) {
      const uint32_t c = cb + static_cast<uint32_t>(lane) / lanes_per_chan;
      A a = A(0), b = A(0);
      if (c < D) {
        const uint32_t lo = c * S;
        const uint32_t p0 = lo / kVec, p1 = (lo + S - 1) / kVec;
#pragma nounroll
        for (uint32_t p = p0 + sub; p <= p1; p += lanes_per_chan) {
          const uint32_t part = p * kVec >= lo ? 0u : 2u;
          a += entries[wave][p][part];
          b += entries[wave][p][part + 1];
        }
      }
      for (uint32_t o = 1; o < lanes_per_chan; o <<= 1) {
        a += __shfl_xor(a, static_cast<int>(o), kWaveSize);
        b += __shfl_xor(b, static_cast<int>(o), kWaveSize);
      }
      if (c < D && sub == 0) {
        A* o = partial + (n * G * D + c0 + c) * 2;
        o[0] = a;
        o[1] = b;
      }
    }
    __threadfence_block();  // the entries are rewritten for the wavefront's next group
  }
}

// --------------------------------------------------------------------------
// General NCHW backward, stage one: per (n, c) row of S contiguous elements,
//   a = sum dy * (x - mu[n, g]),  b = sum dy      -> sums[(n*C + c)*2 + {0,1}]
// One pass over x and dy feeds both the per-group sums (ds, db) and the
// per-channel sums (dgamma, dbeta), which stage two forms from the N*C pairs.
// --------------------------------------------------------------------------
template <typename T, int kTPR, int kVPT, bool kRagged>
__global__ __launch_bounds__(row_threads(kTPR)) void channel_pair_sums_rows(
    const int64_t rows, const int S, const uint32_t D, const T* __restrict__ x,
    const T* __restrict__ dy, const typename IO<T>::Acc* __restrict__ mu,
    typename IO<T>::Acc* __restrict__ sums) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2 * Tile::kSlots];
  const int extent = Tile::extent_of(S);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < rows; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile tx, tg;
    tx.load(x + row * S, extent, A(0));
    tg.load(dy + row * S, extent, A(0));
    const A m = mu[row / D];  // row = n*C + c, so row / D = n*G + g
    A a = A(0), b = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        a += tg.v[i][e] * (tx.v[i][e] - m);  // padding holds dy = 0
        b += tg.v[i][e];
      }
    Tile::reduce_sum_pair(a, b, slots);
    if (Tile::lane() == 0) {
      sums[row * 2] = a;
      sums[row * 2 + 1] = b;
    }
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// Rows longer than the tiles: a 1024-thread workgroup walks the row.
template <typename T>
__global__ __launch_bounds__(kLoopThreads) void channel_pair_sums_looped(
    const int64_t rows, const int64_t S, const uint32_t D, const T* __restrict__ x,
    const T* __restrict__ dy, const typename IO<T>::Acc* __restrict__ mu,
    typename IO<T>::Acc* __restrict__ sums) {
  using A = typename IO<T>::Acc;
  using Loop = RowLoop<T>;
  constexpr int kVec = Loop::kVec;
  __shared__ A slots[2][kLoopWaves];
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const A m = mu[row / D];
    A a = A(0), b = A(0);
    Loop::visit2(x + row * S, dy + row * S, S, A(0),
                 [&](int64_t, const A(&xv)[kVec], const A(&gv)[kVec], int n) {
#pragma unroll
                   for (int e = 0; e < kVec; ++e) {
                     if (e < n) a += gv[e] * (xv[e] - m);
                     b += gv[e];
                   }
                 });
    a = block_allreduce<kLoopWaves>(a, SumOp(), slots[0]);
    b = block_allreduce<kLoopWaves>(b, SumOp(), slots[1]);
    if (threadIdx.x == 0) {
      sums[row * 2] = a;
      sums[row * 2 + 1] = b;
    }
    __syncthreads();
  }
}

// Rows of a few elements (S < 16): one thread per row.
template <typename T>
__global__ __launch_bounds__(256) void channel_pair_sums_short(
    const int64_t rows, const int S, const uint32_t D, const T* __restrict__ x,
    const T* __restrict__ dy, const typename IO<T>::Acc* __restrict__ mu,
    typename IO<T>::Acc* __restrict__ sums) {
  using A = typename IO<T>::Acc;
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; row < rows;
       row += static_cast<int64_t>(gridDim.x) * 256) {
    const A m = mu[row / D];
    A a = A(0), b = A(0);
    for (int j = 0; j < S; ++j) {
      const A g = IO<T>::load1(dy + row * S + j);
      a += g * (IO<T>::load1(x + row * S + j) - m);
      b += g;
    }
    sums[row * 2] = a;
    sums[row * 2 + 1] = b;
  }
}

// The same pairs, and the last step of the general backward, for (n, c) rows of
// up to 1024 elements that are not whole aligned packets (14x14, 7x7 feature
// maps): policies of the LDS-staged short-row kernel (short_rows.h), which
// moves aligned packets whatever S is. The row's scalars are fetched once per
// row with the range's packets.
// The same pairs by the split segment reduction (reduce.h), for long (n, c) rows
// that are too few to give every compute unit a wavefront each: several
// workgroups per row, then `StorePairs` as the second stage's epilogue.
template <typename T>
struct RowPairAccum {
  using A = typename IO<T>::Acc;
  const A* mu;
  uint32_t D;
  A m;
  __device__ __forceinline__ void begin(uint32_t row, uint32_t) { m = mu[row / D]; }
  template <int V>
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, uint32_t, const A (&x)[V],
                                      const A (&dy)[V], A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      a += dy[e] * (x[e] - m);
      b += dy[e];
    }
  }
};
template <typename A>
struct StorePairs {
  A* out;
  __device__ __forceinline__ void operator()(uint32_t o, A a, A b) const {
    out[2 * o] = a;
    out[2 * o + 1] = b;
  }
};
// Rows of more than 1024 elements, fewer than 2048 of them: how many workgroups share one.
inline uint32_t few_long_rows_split(int64_t rows, int64_t S) {
  return rows < 2048 && S > 1024 ? pick_split(rows, S) : 0u;
}

template <typename T, int kE>
struct GroupRowPairSums {  // in0 = x, in1 = dy; reads only
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 1;
  static constexpr bool kReadOnly = true;
  const A* mu;
  uint32_t D;
  A* sums;
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[1]) const { w[0] = mu[row / D]; }
  // the same for the one-wavefront-per-row kernel (long_rows.h)
  static constexpr int kParams = 1;
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[1]) const { fetch_side(row, w); }
  __device__ __forceinline__ void add(const A* w, A x, A dy, A& a, A& b) const {
    a += dy * (x - w[0]);
    b += dy;
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A* side, int, int, A (&x)[kE],
                                      const A (&dy)[kE]) const {
    const A m = side[0];
    A a = A(0), b = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {  // lanes past the row hold dy = 0
      a += dy[j] * (x[j] - m);
      b += dy[j];
    }
    a = group_allreduce<kL>(a, SumOp());
    b = group_allreduce<kL>(b, SumOp());
    if (threadIdx.x % kL == 0) {
      sums[2 * r] = a;
      sums[2 * r + 1] = b;
    }
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

template <typename T, int kE>
struct GroupRowGradMap {  // in0 = x (overwritten with dx), in1 = dy
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 6;
  GroupNormGradApply<T, 1> f;
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  // the terms of GroupNormGradApply::one that depend on the row only
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[6]) const {
    const uint32_t ng = static_cast<uint32_t>(row / f.sh.D);
    const A m = f.mu[ng], r = f.rsig[ng], s = f.ds[ng], b = f.db[ng];
    w[0] = m, w[1] = r, w[2] = b * m - s, w[3] = r * r * r, w[4] = b * r;
    w[5] = f.gamma[row % f.sh.C];
  }
  static constexpr int kParams = 6;
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[6]) const { fetch_side(row, w); }
  __device__ __forceinline__ A apply(const A* w, A x, A dy) const {
    const A u = w[2] * (x - w[0]) * w[3];
    return w[5] * dy * w[1] + (u - w[4]) * f.denom;
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A* w, int, int, A (&x)[kE],
                                      const A (&dy)[kE]) const {
#pragma unroll
    for (int j = 0; j < kE; ++j) x[j] = apply(w, x[j], dy[j]);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

// Workgroups of group_grad_from_channel_sums that form ds / db: a group takes
// D rounded up to a power of two (at most 64) of a workgroup's 256 threads.
inline uint32_t group_sum_blocks(const GroupShape& sh) {
  uint32_t span = 1;
  while (span < sh.D && span < static_cast<uint32_t>(kWaveSize)) span <<= 1;
  return static_cast<uint32_t>(ceil_div(static_cast<int64_t>(sh.N) * sh.G, 256 / span));
}

// Forward of such rows. The map: y = (x - mu) * rsig * gamma + beta with the four
// scalars of the (n, c) row. The statistics: a group is one row of D*S
// elements; sums are shifted by the row's first element.
template <typename T, int kE>
struct GroupRowApply {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 4;
  static constexpr int kParams = 4;
  GroupNormApply<T, 1> f;
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[4]) const {
    const uint32_t ng = static_cast<uint32_t>(row / f.sh.D);
    const uint32_t c = static_cast<uint32_t>(row % f.sh.C);
    w[0] = f.mu[ng], w[1] = f.rsig[ng], w[2] = f.gamma[c], w[3] = f.beta[c];
  }
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[4]) const { fetch_side(row, w); }
  __device__ __forceinline__ A apply(const A* w, A x, A) const {
    return (x - w[0]) * w[1] * w[2] + w[3];
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A* w, int, int, A (&x)[kE],
                                      const A (&)[kE]) const {
#pragma unroll
    for (int j = 0; j < kE; ++j) x[j] = apply(w, x[j], A(0));
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

template <typename T>
struct GroupRowMoments {  // a = sum (x - first), b = sum (x - first)^2 over a group's row
  using A = typename IO<T>::Acc;
  static constexpr int kParams = 1;
  const T* x;
  int64_t L;
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[1]) const {
    w[0] = load_shift(x + row * L);
  }
  __device__ __forceinline__ void add(const A* w, A v, A, A& a, A& b) const {
    const A d = v - w[0];
    a += d;
    b += d * d;
  }
};
template <typename T>
__global__ __launch_bounds__(256) void group_stats_from_row_sums(
    const int64_t rows, const int64_t L, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ pairs, typename IO<T>::Acc* __restrict__ mu,
    typename IO<T>::Acc* __restrict__ rsig) {
  using A = typename IO<T>::Acc;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (row >= rows) return;
  const A inv = A(1) / A(L);
  const A d = pairs[2 * row] * inv;
  mu[row] = load_shift(x + row * L) + d;
  rsig[row] = acc_rsqrt_exact((pairs[2 * row + 1] * inv - d * d) + eps);
}

inline bool ragged_group_rows(const GroupShape& sh, size_t elem_bytes, const void* x,
                              const void* dy, const void* dx) {
  const uint32_t vec = static_cast<uint32_t>(16 / elem_bytes);
  const bool packets = sh.S % vec == 0 && aligned16(x) && aligned16(dy) && aligned16(dx);
  return sh.nchw && !packets && congruent16(x, dy) && congruent16(x, dx);
}
inline bool short_group_rows(const GroupShape& sh, size_t elem_bytes, const void* x,
                             const void* dy, const void* dx) {
  return sh.S <= 1024 && ragged_group_rows(sh, elem_bytes, x, dy, dx);
}
// Longer rows of that kind: one wavefront per (n, c) row (long_rows.h).
inline bool long_group_rows(const GroupShape& sh, size_t elem_bytes, const void* x, const void* dy,
                            const void* dx) {
  return sh.S > 1024 && ragged_group_rows(sh, elem_bytes, x, dy, dx);
}

// Stage two. Workgroups [0, group_blocks) form, one thread per (n, g),
//   ds = sum_c gamma_c * (a_c + mu * b_c),  db = sum_c gamma_c * b_c   over the group's channels;
// the others own 64 adjacent channels each (one per lane), their four
// wavefronts stride over n and are combined in wavefront order:
//   dgamma_c = sum_n a[n, c] * rsig[n, g],  dbeta_c = sum_n b[n, c].
template <typename A>
__global__ __launch_bounds__(256) void group_grad_from_channel_sums(
    const uint32_t N, const uint32_t G, const uint32_t D, const uint32_t group_blocks,
    const A* __restrict__ sums, const A* __restrict__ gamma, const A* __restrict__ mu,
    const A* __restrict__ rsig, A* __restrict__ ds, A* __restrict__ db, A* __restrict__ dgamma,
    A* __restrict__ dbeta) {
  __shared__ A lds[4][kWaveSize][2];
  const uint32_t C = G * D;
  if (blockIdx.x < group_blocks) {
    // `span` adjacent lanes (a power of two, D rounded up, at most 64) share a
    // group: adjacent lanes read adjacent channel pairs.
    uint32_t span = 1;
    while (span < D && span < kWaveSize) span <<= 1;
    const uint32_t per_block = 256 / span;
    const uint32_t ng = blockIdx.x * per_block + threadIdx.x / span;
    const uint32_t l = threadIdx.x % span;
    const bool on = ng < N * G;
    const uint32_t g = on ? ng % G : 0;
    const A m = on ? mu[ng] : A(0);
    const A* row = sums + (static_cast<size_t>(on ? ng / G : 0) * C + g * D) * 2;
    A s = A(0), b = A(0);
    for (uint32_t d = l; d < D; d += span) {
      const A w = gamma[g * D + d];
      s += w * (row[2 * d] + m * row[2 * d + 1]);
      b += w * row[2 * d + 1];
    }
    for (uint32_t o = 1; o < span; o <<= 1) {
      s += __shfl_xor(s, static_cast<int>(o), kWaveSize);
      b += __shfl_xor(b, static_cast<int>(o), kWaveSize);
    }
    if (on && l == 0) {
      ds[ng] = s;
      db[ng] = b;
    }
    return;
  }
  if (dgamma == nullptr) return;
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t c = (blockIdx.x - group_blocks) * kWaveSize + lane;
  A a = A(0), b = A(0);
  if (c < C) {
    const uint32_t g = c / D;
#pragma unroll 8
    for (uint32_t n = wave; n < N; n += 4) {
      const size_t idx = (static_cast<size_t>(n) * C + c) * 2;
      a += sums[idx] * rsig[n * G + g];
      b += sums[idx + 1];
    }
  }
  lds[wave][lane][0] = a;
  lds[wave][lane][1] = b;
  __syncthreads();
  if (wave == 0 && c < C) {
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      a += lds[w][lane][0];
      b += lds[w][lane][1];
    }
    dgamma[c] = a;
    dbeta[c] = b;
  }
}

// --------------------------------------------------------------------------
// NHWC: x is [N, S, C] and a group is D adjacent columns of one sample's
// [S, C] matrix. Stage one reduces every (n, c) column over s with full-width
// row accesses (a lane owns kW adjacent channels: one 16-byte packet, or one
// element for unaligned tensors); a sample's rows are split over `split`
// workgroups. partial[((n*split + k)*C + c)*2 + {0,1}]. F provides
//   void begin(uint32_t n, uint32_t c)
//   void add(A x0, A x1, A& a, A& b)
// --------------------------------------------------------------------------
struct BatchedColumns {
  uint32_t N, S, C, split;
};

template <typename T, int kIn, int kW, typename F>
__global__ __launch_bounds__(kReduceThreads) void reduce2_batched_columns(
    const BatchedColumns d, const T* __restrict__ in0, const T* __restrict__ in1, F f,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds[kReduceWaves][kWaveSize][2 * kW];
  // Lanes along a row: the whole wavefront, or for fewer than 64 * kW columns
  // the power of two that covers a row, the other lane bits taking adjacent rows.
  uint32_t along_lanes = 1;
  while (along_lanes < kWaveSize && along_lanes * kW < d.C) along_lanes <<= 1;
  const uint32_t rows_per_wave = kWaveSize / along_lanes;
  const uint32_t tile_cols = along_lanes * kW;
  const uint32_t tiles = (d.C + tile_cols - 1) / tile_cols;
  const uint32_t tile = blockIdx.x % tiles;
  const uint32_t k = (blockIdx.x / tiles) % d.split;
  const uint32_t n = blockIdx.x / (tiles * d.split);
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t across = lane / along_lanes;
  const uint32_t c0 = tile * tile_cols + (lane % along_lanes) * kW;
  A a[kW], b[kW];
#pragma unroll
  for (int e = 0; e < kW; ++e) a[e] = b[e] = A(0);
  if (c0 < d.C) {
    F fs[kW];
#pragma unroll
    for (int e = 0; e < kW; ++e) {
      fs[e] = f;
      fs[e].begin(n, c0 + e);
    }
    const uint32_t base = n * d.S * d.C + c0;
#pragma unroll 4
    for (uint32_t r = (k * kReduceWaves + wave) * rows_per_wave + across; r < d.S;
         r += d.split * kReduceWaves * rows_per_wave) {
      const uint32_t off = base + r * d.C;
      A x0[kW], x1[kW];
      if constexpr (kW == 1) {
        x0[0] = IO<T>::load1(in0 + off);
        x1[0] = kIn == 2 ? IO<T>::load1(in1 + off) : A(0);
      } else {
        load_unpack_keep<T>(in0 + off, x0);
        if constexpr (kIn == 2) load_unpack_keep<T>(in1 + off, x1);
      }
#pragma unroll
      for (int e = 0; e < kW; ++e) fs[e].add(x0[e], kIn == 2 ? x1[e] : A(0), a[e], b[e]);
    }
  }
  for (uint32_t o = along_lanes; o < kWaveSize; o <<= 1) {  // the lanes that share a column
#pragma unroll
    for (int e = 0; e < kW; ++e) {
      a[e] += __shfl_xor(a[e], static_cast<int>(o), kWaveSize);
      b[e] += __shfl_xor(b[e], static_cast<int>(o), kWaveSize);
    }
  }
#pragma unroll
  for (int e = 0; e < kW; ++e) {
    lds[wave][lane][2 * e] = a[e];
    lds[wave][lane][2 * e + 1] = b[e];
  }
  __syncthreads();
  if (wave == 0 && across == 0 && c0 < d.C) {
    A* out = partial + ((static_cast<size_t>(n) * d.split + k) * d.C + c0) * 2;
#pragma unroll
    for (int e = 0; e < kW; ++e) {
#pragma unroll
      for (int w = 1; w < kReduceWaves; ++w) {
        a[e] += lds[w][lane][2 * e];
        b[e] += lds[w][lane][2 * e + 1];
      }
      out[2 * e] = a[e];
      out[2 * e + 1] = b[e];
    }
  }
}

// Rows of one sample per stage-one workgroup: enough workgroups to fill the
// device, at least ~64 rows each.
inline uint32_t batched_split(int64_t N, int64_t S, int64_t C, int kw) {
  const int64_t tiles = ceil_div(C, kWaveSize * kw);
  int64_t split = ceil_div(static_cast<int64_t>(num_cus()) * 8, N * tiles);
  const int64_t by_work = ceil_div(S, 64);
  if (split > by_work) split = by_work;
  if (split < 1) split = 1;
  if (split > 256) split = 256;
  return static_cast<uint32_t>(split);
}
// Largest scratch either variant (packet or scalar lanes) needs, in pairs.
inline size_t batched_partial_pairs(int64_t N, int64_t S, int64_t C) {
  uint32_t split = batched_split(N, S, C, 1);
  const uint32_t split8 = batched_split(N, S, C, 8);
  if (split8 > split) split = split8;
  return static_cast<size_t>(N) * split * C;
}

template <typename T>
struct ColumnStatsAccum {  // sums shifted by the column's first element
  using A = typename IO<T>::Acc;
  const T* x;
  uint32_t S, C;
  A shift;
  __device__ __forceinline__ void begin(uint32_t n, uint32_t c) {
    shift = load_shift(x + static_cast<size_t>(n) * S * C + c);
  }
  __device__ __forceinline__ void add(A x0, A, A& a, A& b) const {
    const A d = x0 - shift;
    a += d;
    b += d * d;
  }
};

template <typename T>
struct ColumnPairAccum {  // a = sum dy * (x - mu[n, g]), b = sum dy
  using A = typename IO<T>::Acc;
  const A* mu;
  uint32_t G, D;
  A m;
  __device__ __forceinline__ void begin(uint32_t n, uint32_t c) { m = mu[n * G + c / D]; }
  __device__ __forceinline__ void add(A x0, A dy, A& a, A& b) const {
    a += dy * (x0 - m);
    b += dy;
  }
};

// Last stage of the NHWC statistics, one thread per (n, g), from the per-(n, c)
// pairs: per channel mean_c = shift_c + a_c/S and M2_c = b_c - a_c^2/S, combined
// over the group's D channels as mean = avg(mean_c),
// M2 = sum(M2_c + S*(mean_c - mean)^2).
template <typename T>
__global__ __launch_bounds__(256) void group_stats_from_column_sums(
    const BatchedColumns d, const uint32_t G, const uint32_t D, const typename IO<T>::Acc eps,
    const T* __restrict__ x, const typename IO<T>::Acc* __restrict__ sums,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig) {
  using A = typename IO<T>::Acc;
  const uint32_t ng = blockIdx.x * 256 + threadIdx.x;
  if (ng >= d.N * G) return;
  const uint32_t n = ng / G, g = ng - n * G;
  const A inv_s = A(1) / A(d.S);
  const T* first_row = x + static_cast<size_t>(n) * d.S * d.C + g * D;
  const A* pairs = sums + (static_cast<size_t>(n) * d.C + g * D) * 2;
  A mean = A(0);
#pragma unroll 8
  for (uint32_t j = 0; j < D; ++j) mean += IO<T>::load1(first_row + j) + pairs[2 * j] * inv_s;
  mean = mean / A(D);
  A m2 = A(0);
#pragma unroll 8
  for (uint32_t j = 0; j < D; ++j) {
    const A a = pairs[2 * j], b = pairs[2 * j + 1];
    const A dm = IO<T>::load1(first_row + j) + a * inv_s - mean;
    m2 += (b - a * a * inv_s) + A(d.S) * dm * dm;
  }
  mu[ng] = mean;
  rsig[ng] = acc_rsqrt_exact(m2 / (A(D) * A(d.S)) + eps);
}

// sums[(n*C + c)*2 + {0,1}] = sum over the `split` partial pairs of (n, c).
template <typename A>
__global__ __launch_bounds__(256) void sum_batched_partials(const BatchedColumns d,
                                                            const A* __restrict__ partial,
                                                            A* __restrict__ sums) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= d.N * d.C) return;
  const uint32_t n = i / d.C, c = i - n * d.C;
  A a = A(0), b = A(0);
#pragma unroll 16
  for (uint32_t k = 0; k < d.split; ++k) {  // independent loads: issued sixteen at a time
    const size_t idx = ((static_cast<size_t>(n) * d.split + k) * d.C + c) * 2;
    a += partial[idx];
    b += partial[idx + 1];
  }
  sums[static_cast<size_t>(i) * 2] = a;
  sums[static_cast<size_t>(i) * 2 + 1] = b;
}

template <typename T, int kIn, typename F>
BatchedColumns launch_batched_columns(const GroupShape& sh, const T* in0, const T* in1, F f,
                                      typename IO<T>::Acc* partial, hipStream_t stream) {
  constexpr int kVec = IO<T>::kVec;
  const bool packets = sh.C % kVec == 0 && aligned16(in0) && (kIn == 1 || aligned16(in1));
  BatchedColumns d{sh.N, sh.S, sh.C, 1};
  if (packets) {
    d.split = batched_split(sh.N, sh.S, sh.C, kVec);
    const uint32_t tiles = static_cast<uint32_t>(ceil_div(sh.C, kWaveSize * kVec));
    hipLaunchKernelGGL((reduce2_batched_columns<T, kIn, kVec, F>), dim3(sh.N * d.split * tiles),
                       dim3(kReduceThreads), 0, stream, d, in0, in1, f, partial);
  } else {
    d.split = batched_split(sh.N, sh.S, sh.C, 1);
    const uint32_t tiles = static_cast<uint32_t>(ceil_div(sh.C, kWaveSize));
    hipLaunchKernelGGL((reduce2_batched_columns<T, kIn, 1, F>), dim3(sh.N * d.split * tiles),
                       dim3(kReduceThreads), 0, stream, d, in0, in1, f, partial);
  }
  return d;
}

// Sums P partial rows of 2*C interleaved (dgamma, dbeta) words. A workgroup of
// 16 wavefronts owns 64 adjacent words; wavefront w adds rows w, w+16, ...
template <typename A>
__global__ __launch_bounds__(1024) void sum_partial_rows(const uint32_t P, const uint32_t C,
                                                         const A* __restrict__ partial,
                                                         A* __restrict__ dgamma,
                                                         A* __restrict__ dbeta) {
  __shared__ A lds[16][kWaveSize];
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const uint32_t word = blockIdx.x * kWaveSize + lane;
  const uint32_t words = 2 * C;
  A acc = A(0);
  if (word < words) {
#pragma unroll 8
    for (uint32_t p = wave; p < P; p += 16) acc += partial[static_cast<size_t>(p) * words + word];
  }
  lds[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && word < words) {
#pragma unroll
    for (int w = 1; w < 16; ++w) acc += lds[w][lane];
    if (word & 1) {
      dbeta[word >> 1] = acc;
    } else {
      dgamma[word >> 1] = acc;
    }
  }
}

// The same for rows of whole 16-byte packets (C even for fp32: a packet holds
// the (dgamma, dbeta) pairs of two adjacent columns, or one pair of doubles).
// A workgroup owns kLanes adjacent packets of every partial row; its
// 1024 / kLanes lane groups take rows g, g + groups, ..., several loads in
// flight per lane, and are added up through LDS in a fixed order. kLanes is 32
// (512 contiguous bytes per row) for the widest rows, 16 for rows of up to 4096
// packets and 8 (one cache line) for narrow ones, which would otherwise leave
// all but a few compute units idle.
template <typename A, int kLanes>
__global__ __launch_bounds__(1024) void sum_partial_rows_packets(const uint32_t P, const uint32_t C,
                                                                 const A* __restrict__ partial,
                                                                 A* __restrict__ dgamma,
                                                                 A* __restrict__ dbeta) {
  constexpr int kPer = 16 / sizeof(A);  // words per packet
  constexpr int kGroups = 1024 / kLanes;
  constexpr int kWords = kLanes * kPer;  // words of the result a workgroup owns
  constexpr int kParts = 1024 / kWords < 8 ? 1024 / kWords : 8;
  __shared__ A lds[kGroups][kWords];
  __shared__ A parts[kParts][kWords];
  const uint32_t lane = threadIdx.x % kLanes;
  const uint32_t group = threadIdx.x / kLanes;
  const uint32_t packets = 2 * C / kPer;
  const uint32_t packet = blockIdx.x * kLanes + lane;
  A acc[kPer];
#pragma unroll
  for (int e = 0; e < kPer; ++e) acc[e] = A(0);
  if (packet < packets) {
    const A* col = partial + static_cast<size_t>(packet) * kPer;
#pragma unroll 4
    for (uint32_t p = group; p < P; p += kGroups) {
      A v[kPer];
      IO<A>::unpack(load_packet(col + static_cast<size_t>(p) * 2 * C), v);
#pragma unroll
      for (int e = 0; e < kPer; ++e) acc[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < kPer; ++e) lds[group][lane * kPer + e] = acc[e];
  __syncthreads();
  // kParts threads per word each add a run of the lane groups, then one thread adds the runs
  if (threadIdx.x < kParts * kWords) {
    const uint32_t w = threadIdx.x % kWords, part = threadIdx.x / kWords;
    constexpr int kRun = kGroups / kParts;
    A t = lds[part * kRun][w];
#pragma unroll 8
    for (int g = 1; g < kRun; ++g) t += lds[part * kRun + g][w];
    parts[part][w] = t;
  }
  __syncthreads();
  if (threadIdx.x < kWords) {
    const uint32_t word = blockIdx.x * kWords + threadIdx.x;
    A total = parts[0][threadIdx.x];
#pragma unroll
    for (int q = 1; q < kParts; ++q) total += parts[q][threadIdx.x];
    if (word < 2 * C) {
      if (word & 1) {
        dbeta[word >> 1] = total;
      } else {
        dgamma[word >> 1] = total;
      }
    }
  }
}

template <typename A>
void launch_sum_partial_rows(uint32_t P, uint32_t C, const A* partial, A* dgamma, A* dbeta,
                             hipStream_t stream) {
  constexpr uint32_t kPer = 16 / sizeof(A);
  const uint32_t packets = 2 * C / kPer;
  if ((2 * C) % kPer != 0 || !aligned16(partial)) {
    hipLaunchKernelGGL((sum_partial_rows<A>), dim3(static_cast<unsigned>(ceil_div(2 * C, kWaveSize))),
                       dim3(1024), 0, stream, P, C, partial, dgamma, dbeta);
  } else if (packets > 4096) {
    hipLaunchKernelGGL((sum_partial_rows_packets<A, 32>),
                       dim3(static_cast<unsigned>(ceil_div(packets, 32))), dim3(1024), 0, stream, P,
                       C, partial, dgamma, dbeta);
  } else if (packets > 1024) {
    // 128 to 256 workgroups: measured on MI355X at C = 4096 (2048 packets), 32 lanes per row
    // chunk (64 workgroups) take 0.4-1 us longer than 16 or 8
    hipLaunchKernelGGL((sum_partial_rows_packets<A, 16>),
                       dim3(static_cast<unsigned>(ceil_div(packets, 16))), dim3(1024), 0, stream, P,
                       C, partial, dgamma, dbeta);
  } else {
    hipLaunchKernelGGL((sum_partial_rows_packets<A, 8>),
                       dim3(static_cast<unsigned>(ceil_div(packets, 8))), dim3(1024), 0, stream, P, C,
                       partial, dgamma, dbeta);
  }
}

struct RowGradPlan {
  bool use_rows;
  RowConfig cfg;
  int threads;  // workgroup size: 512 (two per compute unit) or 1024 (one)
  unsigned grid;
  bool ragged;  // rows that are not whole packets
};

// Tiles of the fused row path: the fewest threads per row that hold it with at
// most 16 elements per thread (two raw tiles for the current row, two for the
// prefetched one and two accumulator sets must fit 128 registers).
template <typename T>
RowGradPlan plan_row_grad(int64_t N, int64_t G, int64_t D, int64_t S) {
  RowGradPlan p = {false, {0, 0}, 512, 0, false};
  if (G != 1 || S != 1) return p;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kMaxVpt = kVec == 8 ? 2 : 4;
  // staged gamma, padded to whole packets of the row
  if (static_cast<size_t>(ceil_div(D, kVec) * kVec) * sizeof(typename IO<T>::Acc) >
      kMaxStagedParamBytes / 2) {
    return p;
  }
  p.ragged = D % kVec != 0;
  static const RowConfig table[] = {{64, 1},  {64, 2},  {256, 1},  {256, 2},  {512, 1},
                                    {512, 2}, {1024, 1}, {768, 2}, {1024, 2}, {1024, 4}};
  bool found = false;
  for (const RowConfig& c : table) {
    // 16-bit rows of 513 to 1024 packets: one packet per thread of a 1024-thread
    // tile keeps two rows in flight ahead of the current one, which two packets
    // per thread of a 512-thread tile cannot within 128 registers ([8192, 8192]
    // bf16: 73 us against 81 us on MI355X).
    if (kVec == 8 && c.tpr == 512 && c.vpt == 2) continue;
    if (!found && c.vpt <= kMaxVpt && ceil_div(D, kVec) <= static_cast<int64_t>(c.tpr) * c.vpt) {
      p.cfg = c;
      found = true;
    }
  }
  if (!found) return p;
  p.threads = p.cfg.tpr >= 768 ? p.cfg.tpr : 512;
  // Rows of 2049 to 4096 elements: 1024-thread workgroups (four 16-bit rows on 256
  // threads each, two wider ones on 512) instead of two 512-thread workgroups per
  // compute unit. Half as many partial dgamma / dbeta rows leave the kernel and enter
  // the second stage ([8192, 4096]: bf16 38 us against 40 us, fp32 67 us against 69 us;
  // [16384, 4096] fp32 151 us against 169 us).
  if (p.cfg.vpt == 2 && ((p.cfg.tpr == 256 && kVec == 8) || (p.cfg.tpr == 512 && kVec < 8))) {
    p.threads = 1024;
  }
  // Wider rows of 4- or 8-byte elements (more than 704 packets, e.g. 3072 to 4096 floats):
  // one 512-thread workgroup per compute unit, i.e. one row at a time with two rows
  // requested ahead, instead of two rows at a time on 1024 threads. Fewer bytes in flight
  // per compute unit stream better here, and the partial rows stay at one per compute unit
  // (fp32 [8192, 4096] row kernel 70.6 -> 68.0 us, [32768, 4096] 280 -> 261 us on MI355X;
  // at 2560 floats the two-row tile is ahead, 45.1 against 46.2 us).
  bool one_per_cu = false;
  if (p.cfg.tpr == 512 && p.cfg.vpt == 2 && kVec < 8 && ceil_div(D, kVec) > 704) {
    p.threads = 512;
    one_per_cu = true;
  }
  const int per_cu = p.threads == 512 && !one_per_cu ? 2 : 1;
  const int64_t groups = p.threads / p.cfg.tpr;
  const int64_t want = ceil_div(N, groups);
  const int64_t cap = num_cus() * per_cu;
  p.grid = static_cast<unsigned>(want < cap ? want : cap);
  p.use_rows = true;
  return p;
}

// Fused group backward applies to NCHW groups that fit a multi-wave register
// tile and whose channels are whole packets: 64 or more of them (`mode` tells
// whether they are whole wavefronts of packets), or a power of two below 64.
template <typename T>
bool plan_group_grad_rows(int64_t G, int64_t D, int64_t S, int layout, RowConfig* cfg, int* mode) {
  constexpr int kVec = IO<T>::kVec;
  if (layout != DRAGON_HIP_NCHW || G * D == 1) return false;
  static const RowConfig table[] = {{256, 2}, {256, 4}, {256, 8}, {1024, 4}, {1024, 8}};
  // (512 threads, two workgroups per compute unit at 128 registers, where 1024 threads with four
  // packets each leave room for one; not for the entry-per-packet flavour)
  static const RowConfig table512[] = {{256, 2}, {256, 4}, {256, 8}, {512, 8}, {1024, 8}};
  const int64_t per_chan = S / kVec;
  if (S % kVec == 0 && per_chan >= kWaveSize) {
    *mode = per_chan % kWaveSize == 0 ? kChannelWaves : kChannelStraddles;
  } else if (S % kVec == 0 && (per_chan & (per_chan - 1)) == 0) {
    *mode = kChannelLanes;
  } else if (S >= kWaveSize * kVec && (D * S) % kVec == 0) {
    // channels of 64 packets' worth or more that are not whole packets
    *mode = kChannelStraddlesAny;
  } else if (S >= kVec && (D * S) % kVec == 0 && D * S / kVec <= kMaxEntryPackets) {
    // channels that are not whole packets (or a number of packets the lane
    // flavour does not take): one LDS entry per packet
    *mode = kChannelPackets;
  } else {
    return false;
  }
  const int64_t npackets = D * S / kVec;
  if (npackets <= kWaveSize * 2) return false;  // a wavefront or two: the general path
  for (const RowConfig& c : *mode == kChannelPackets || sizeof(T) > 4 ? table : table512) {
    if (npackets <= static_cast<int64_t>(c.tpr) * c.vpt) {
      *cfg = c;
      return true;
    }
  }
  return false;
}

// The most workgroups the NHWC sample backward (group_norm_grad_nhwc_samples) is
// launched with: sizes its partial rows.
inline uint32_t nhwc_sample_rows(int64_t N) {
  const int64_t cap = static_cast<int64_t>(num_cus()) * 4;
  return static_cast<uint32_t>(N < cap ? N : cap);
}

template <typename T>
size_t group_norm_grad_scratch(int64_t N, int64_t G, int64_t D, int64_t S, int layout) {
  using A = typename IO<T>::Acc;
  const RowGradPlan rp = plan_row_grad<T>(N, G, D, S);
  // LayerNorm backward: one partial (dgamma, dbeta) row per workgroup of the row
  // kernels, or of the staged short-row kernel when the addresses select it
  size_t row_paths = rp.use_rows ? static_cast<size_t>(rp.grid) * D * 2 * sizeof(A) : 0;
  if (G == 1 && S == 1 && D <= 1024) {
    const size_t staged = static_cast<size_t>(short_grad_max_grid()) * D * 2 * sizeof(A);
    if (staged > row_paths) row_paths = staged;
  }
  if (rp.use_rows) return row_paths;
  if (G == 1 && S == 1) {
    // wide rows: the packet or the element flavour, by the addresses
    const size_t packets = wide_grad_words(N, D, IO<T>::kVec), elems = wide_grad_words(N, D, 1);
    return (packets > elems ? packets : elems) * sizeof(A);
  }
  const int64_t C = G * D;
  // per-(n, c) pairs of the fused and the general path; NHWC adds the stage-one partial pairs
  size_t pairs = static_cast<size_t>(N) * C;
  if (pairs * 2 * sizeof(A) < row_paths) pairs = row_paths / (2 * sizeof(A));
  if (layout != DRAGON_HIP_NCHW) {
    pairs += batched_partial_pairs(N, S, C);
    // or one partial (dgamma, dbeta) row per workgroup of the sample kernel
    const size_t sample_pairs = static_cast<size_t>(nhwc_sample_rows(N)) * C;
    if (pairs < sample_pairs) pairs = sample_pairs;
  }
  // few long rows: the split reduction's partial pairs behind the N*C pairs
  if (layout == DRAGON_HIP_NCHW) pairs += static_cast<size_t>(N) * C * few_long_rows_split(N * C, S);
  size_t bytes = pairs * 2 * sizeof(A);
  // the slice path: the exchange of K pairs per group, then one pair per wavefront block
  if (layout == DRAGON_HIP_NCHW && S % (IO<T>::kVec * kWaveSize) == 0) {
    const uint32_t L = static_cast<uint32_t>(D * S);
    const SliceUnits u{static_cast<uint32_t>(N * G), 1u, L, L, L};
    const CoopPlan p = plan_coop<T>(u, 2);
    if (p.ok) {
      const size_t slices = coop_exchange_bytes(static_cast<size_t>(u.units) * p.K, sizeof(A)) +
          static_cast<size_t>(N) * C * (S / IO<T>::kVec / kWaveSize) * 2 * sizeof(A);
      if (slices > bytes) bytes = slices;
    }
  }
  return bytes;
}

// --------------------------------------------------------------------------
// NCHW groups too large for one workgroup's registers: the slice kernel
// (slices.h) with the group as the reduction unit, one run of D*S elements.
// --------------------------------------------------------------------------
inline SliceUnits group_units(const GroupShape& sh) {
  const uint32_t L = sh.D * sh.S;
  return SliceUnits{sh.N * sh.G, 1u, L, L, L};
}

// Moments -> InvStd -> GroupNorm with x read once.
template <typename T>
struct GroupSlicesForward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr bool kBeginReadsInput = true;
  using Merge = PairSum;
  A inv_l, eps;
  const A* gamma;
  const A* beta;
  A* mu;
  A* rsig;
  uint32_t G, D, packets_per_chan;
  A shift, mean, rs;
  __device__ __forceinline__ void begin(uint32_t, uint32_t base, const T* x) {
    shift = load_shift(x + base);  // one sample of the group
  }
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t, uint32_t, const A (&x)[V], const A (&)[V],
                                             A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const A t = x[e] - shift;
      a += t;
      b += t * t;
    }
  }
  __device__ __forceinline__ void finish(uint32_t row, bool leader, A a, A b) {
    const A dm = a * inv_l;
    mean = shift + dm;
    const A var = b * inv_l - dm * dm;
    rs = acc_rsqrt_exact(var + eps);
    if (leader) {
      mu[row] = mean;
      rsig[row] = rs;
    }
  }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t row, uint32_t j, A (&x)[V], const A (&)[V]) const {
    const uint32_t c = (row % G) * D + j / packets_per_chan;
    const A gs = gamma[c] * rs, bc = beta[c];
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = (x[e] - mean) * gs + bc;
  }
};

// GroupNormGrad with x and dy read once. The sums exchanged between the slices
// are the group's ds and db; a wavefront's 64 packets lie in one channel
// (S / kVec is a multiple of 64), so its share of that channel's dgamma / dbeta
// is one wave reduction, written to chan_part[(row * blocks + j / 64) * 2] and
// summed per channel by a second, small kernel.
template <typename T>
struct GroupSlicesBackward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  using Merge = PairSum;
  A denom;  // 1 / (D * S)
  const A* mu;
  const A* rsig;
  const A* gamma;
  A* ds;
  A* db;
  A* chan_part;
  uint32_t G, D, packets_per_chan, blocks_per_row;
  A m, r, u0, v0;
  __device__ __forceinline__ void begin(uint32_t row, uint32_t, const T*) { m = mu[row], r = rsig[row]; }
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t row, uint32_t j, const A (&x)[V],
                                             const A (&dy)[V], A& a, A& b) const {
    const A g = gamma[(row % G) * D + j / packets_per_chan];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const A t = g * dy[e];
      a += t * x[e];
      b += t;
    }
  }
  __device__ __forceinline__ void finish(uint32_t row, bool leader, A a, A b) {
    if (leader) {
      ds[row] = a;
      db[row] = b;
    }
    u0 = (b * m - a) * (r * r * r) * denom;
    v0 = b * r * denom;
  }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t row, uint32_t j, A (&x)[V],
                                            const A (&dy)[V]) const {
    const A gr = gamma[(row % G) * D + j / packets_per_chan] * r;
    A t1 = A(0), t2 = A(0);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const A xc = x[e] - m;
      t1 += dy[e] * xc * r;
      t2 += dy[e];
      x[e] = gr * dy[e] + (u0 * xc - v0);
    }
    t1 = wave_allreduce(t1, SumOp());
    t2 = wave_allreduce(t2, SumOp());
    if ((threadIdx.x & (kWaveSize - 1)) == 0) {
      A* o = chan_part + (static_cast<size_t>(row) * blocks_per_row + j / kWaveSize) * 2;
      o[0] = t1;
      o[1] = t2;
    }
  }
};

// dgamma[c], dbeta[c] = sum over n and over the wavefront blocks of channel (n, c).
template <typename A>
__global__ __launch_bounds__(kReduceThreads) void sum_channel_blocks(
    const uint32_t N, const uint32_t C, const uint32_t blocks_per_chan, const A* __restrict__ part,
    A* __restrict__ dgamma, A* __restrict__ dbeta) {
  __shared__ A lds[2 * kReduceWaves];
  const uint32_t c = blockIdx.x;
  A a = A(0), b = A(0);
  for (uint32_t i = threadIdx.x; i < N * blocks_per_chan; i += kReduceThreads) {
    const uint32_t n = i / blocks_per_chan, e = i - n * blocks_per_chan;
    const A* p = part + ((static_cast<size_t>(n) * C + c) * blocks_per_chan + e) * 2;
    a += p[0];
    b += p[1];
  }
  block_reduce_pair(a, b, lds);
  if (threadIdx.x == 0) {
    dgamma[c] = a;
    dbeta[c] = b;
  }
}

// Pairs of scratch the backward needs beyond the slices' own: one per wavefront block.
template <typename T>
size_t group_slices_block_pairs(const GroupShape& sh) {
  return static_cast<size_t>(sh.N) * sh.C * (sh.S / IO<T>::kVec / kWaveSize);
}

template <typename T>
int try_group_norm_grad_slices(const GroupShape& sh, const void* x, const void* mu, const void* rsig,
                               const void* gamma, const void* dy, void* ds, void* db, void* dgamma,
                               void* dbeta, void* dx, void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  if (!sh.nchw || sh.S % (kVec * kWaveSize) != 0) return kNotApplicable;
  const SliceUnits u = group_units(sh);
  const CoopPlan p = plan_coop<T>(u, 2);
  if (!p.ok) return kNotApplicable;
  A* pairs = static_cast<A*>(scratch);
  A* chan_part = reinterpret_cast<A*>(
      static_cast<char*>(scratch) +
      coop_exchange_bytes(static_cast<size_t>(u.units) * p.K, sizeof(A)));
  const uint32_t blocks_per_chan = sh.S / kVec / kWaveSize;
  const GroupSlicesBackward<T> op{A(1) / A(static_cast<int64_t>(sh.D) * sh.S),
                                  static_cast<const A*>(mu),
                                  static_cast<const A*>(rsig),
                                  static_cast<const A*>(gamma),
                                  static_cast<A*>(ds),
                                  static_cast<A*>(db),
                                  chan_part,
                                  sh.G,
                                  sh.D,
                                  sh.S / kVec,
                                  sh.D * blocks_per_chan,
                                  A(0), A(0), A(0), A(0)};
  const int st = try_channel_slices<T>(u, op, static_cast<const T*>(x), static_cast<const T*>(dy),
                                       static_cast<T*>(dx), pairs, stream);
  if (st != DRAGON_HIP_OK) return st;
  hipLaunchKernelGGL((sum_channel_blocks<A>), dim3(sh.C), dim3(kReduceThreads), 0, stream, sh.N, sh.C,
                     blocks_per_chan, chan_part, static_cast<A*>(dgamma), static_cast<A*>(dbeta));
  return status_of_launch();
}

template <typename T>
int try_group_norm_forward_slices(const GroupShape& sh, float eps, const void* x, const void* gamma,
                                  const void* beta, void* mu, void* rsig, void* y, void* scratch,
                                  size_t scratch_bytes, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  if (!sh.nchw || sh.S % kVec != 0) return kNotApplicable;
  const SliceUnits u = group_units(sh);
  if (!plan_coop<T>(u, 1).ok) return kNotApplicable;
  if (!scratch || scratch_bytes < coop_scratch_bytes<T>(u)) return DRAGON_HIP_ESCRATCH;
  const GroupSlicesForward<T> op{A(1) / A(static_cast<int64_t>(sh.D) * sh.S),
                                 A(eps),
                                 static_cast<const A*>(gamma),
                                 static_cast<const A*>(beta),
                                 static_cast<A*>(mu),
                                 static_cast<A*>(rsig),
                                 sh.G,
                                 sh.D,
                                 sh.S / kVec,
                                 A(0), A(0), A(0)};
  const T* xp = static_cast<const T*>(x);
  return try_channel_slices<T>(u, op, xp, xp, static_cast<T*>(y), static_cast<A*>(scratch), stream);
}

inline size_t group_slices_scratch_bytes(int dtype, const GroupShape& sh) {
  if (!sh.nchw) return 0;
  const SliceUnits u = group_units(sh);
  switch (dtype) {
    case DRAGON_HIP_F16: return sh.S % 8 == 0 ? coop_scratch_bytes<f16_t>(u) : 0;
    case DRAGON_HIP_BF16: return sh.S % 8 == 0 ? coop_scratch_bytes<bf16_t>(u) : 0;
    case DRAGON_HIP_F32: return sh.S % 4 == 0 ? coop_scratch_bytes<float>(u) : 0;
    case DRAGON_HIP_F64: return sh.S % 2 == 0 ? coop_scratch_bytes<double>(u) : 0;
    default: return 0;
  }
}

// Groups of up to 1024 elements (a few channels on 14x14, 8x8 or 7x7 maps) as a
// policy of the LDS-staged short-row kernel (short_rows.h): several groups per
// wavefront instead of one group on a fraction of a wavefront's lanes. The
// channel of each of a lane's elements, relative to the group's first channel,
// is the same for every group and is found once; gamma / beta are fetched per
// group.
template <typename T, int kE>
struct GroupShortForward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  A inv_l, eps;
  const A* gamma;
  const A* beta;
  A* mu;
  A* rsig;
  uint32_t G, D, S;
  uint32_t chan[kE];
  __device__ __forceinline__ void set_packed(bool) {}
  template <int kL>
  static constexpr bool packed_ok() { return false; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int l, int) {
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const uint32_t c = static_cast<uint32_t>(l + j * kL) / S;
      chan[j] = c < D ? c : D - 1;  // lanes past the group
    }
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A*, int l, int L, A (&v)[kE],
                                      const A (&)[kE]) const {
    A s = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) s += v[j];  // lanes past the group hold 0
    const A mean = group_allreduce<kL>(s, SumOp()) * inv_l;
    A q = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const A d = v[j] - mean;
      q += l + j * kL < L ? d * d : A(0);
    }
    const A rs = acc_rsqrt_exact(group_allreduce<kL>(q, SumOp()) * inv_l + eps);
    if (l == 0) {
      mu[r] = mean;
      rsig[r] = rs;
    }
    const uint32_t c0 = static_cast<uint32_t>(r % G) * D;
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      v[j] = (v[j] - mean) * (gamma[c0 + chan[j]] * rs) + beta[c0 + chan[j]];
    }
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

// The backward of such groups the same way (x and dy staged). ds / db are
// reductions over the group's lanes; a channel's dgamma / dbeta share is the
// sum over the lane's elements of that channel, one pair of reductions per
// channel of the group (a few channels: D <= 8), written to
// partial[(n*C + c)*2 + {0,1}] as by the row kernels.
template <typename T, int kE>
struct GroupShortBackward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  A denom;
  const A* gamma;
  const A* mu;
  const A* rsig;
  A* ds;
  A* db;
  A* partial;
  uint32_t G, D, S;
  uint32_t chan[kE];
  __device__ __forceinline__ void set_packed(bool) {}
  template <int kL>
  static constexpr bool packed_ok() { return false; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int l, int) {
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const uint32_t c = static_cast<uint32_t>(l + j * kL) / S;
      chan[j] = c < D ? c : D - 1;  // lanes past the group (their dy is 0)
    }
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A*, int l, int, A (&x)[kE],
                                      const A (&dy)[kE]) const {
    const A m = mu[r], rs = rsig[r];
    const uint32_t c0 = static_cast<uint32_t>(r % G) * D;
    A g[kE];
    A s1 = A(0), s2 = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      g[j] = gamma[c0 + chan[j]];
      const A t = g[j] * dy[j];
      s1 += t * x[j];
      s2 += t;
    }
    s1 = group_allreduce<kL>(s1, SumOp());
    s2 = group_allreduce<kL>(s2, SumOp());
    if (l == 0) {
      ds[r] = s1;
      db[r] = s2;
    }
    A* o = partial + (static_cast<size_t>(r / G) * G * D + c0) * 2;
    for (uint32_t d = 0; d < D; ++d) {
      A h1 = A(0), h2 = A(0);
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const bool mine = chan[j] == d;
        h1 += mine ? dy[j] * (x[j] - m) * rs : A(0);
        h2 += mine ? dy[j] : A(0);
      }
      h1 = group_allreduce<kL>(h1, SumOp());
      h2 = group_allreduce<kL>(h2, SumOp());
      if (l == 0) {
        o[2 * d] = h1;
        o[2 * d + 1] = h2;
      }
    }
    const A u0 = (s2 * m - s1) * (rs * rs * rs);
    const A v0 = s2 * rs;
#pragma unroll
    for (int j = 0; j < kE; ++j) x[j] = g[j] * dy[j] * rs + (u0 * (x[j] - m) - v0) * denom;
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

// Fused forward: true when the register-resident kernel was launched.
template <typename T>
bool try_group_norm_forward_rows(const GroupShape& sh, float eps, const void* x, const void* gamma,
                                 const void* beta, void* mu, void* rsig, void* y,
                                 hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  RowConfig cfg;
  const int64_t L = static_cast<int64_t>(sh.D) * sh.S;
  if (!sh.nchw || !pick_row_config(ceil_div(L, kVec), 8, &cfg)) return false;
  const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
  // Groups of at most 32 packets leave half of a wavefront's lanes or more idle in
  // the row kernels: several groups per wavefront, staged through LDS (fp16
  // [4096,96,8,8] 44 -> 31 us, bf16 [4096,64,8,8] 42 -> 21 us; from 49 packets on
  // the row kernels are ahead).
  if (ShortPlan sp; sizeof(T) <= 4 && ceil_div(L, kVec) <= 32 && rows >= 4096 && congruent16(x, y) &&
                    plan_short_rows(L, sizeof(T), 4, aligned16(x), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16;
    const T* xp = static_cast<const T*>(x);
    DRAGON_HIP_SHORT_LAUNCH(T, GroupShortForward, sp, lds, short_grid(rows, sp.rows_per_chunk),
                            stream, rows, static_cast<int>(L), xp, xp, static_cast<T*>(y),
                            A(1) / A(L), A(eps), static_cast<const A*>(gamma),
                            static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig),
                            sh.G, sh.D, sh.S, {});
    return true;
  }
  if (L % kVec != 0 || !aligned16(x) || !aligned16(y)) {
    if (RowConfig wc; sizeof(T) <= 4 && congruent16(x, y) && pick_row_config(L / kVec + 2, 8, &wc)) {
      // the aligned packets that cover each group
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    hipLaunchKernelGGL((group_norm_forward_rows_windows<T, TPR, VPT>),                          \
                       dim3(row_grid(rows, Tile::kRowsPerBlock)), dim3(Tile::kThreads), 0,      \
                       stream, rows, static_cast<int>(L), sh.G, sh.D, sh.S, A(eps),             \
                       static_cast<const T*>(x), static_cast<const A*>(gamma),                  \
                       static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig), \
                       static_cast<T*>(y));                                                     \
  }
      DRAGON_HIP_ROW_SWITCH(wc, LAUNCH);
#undef LAUNCH
      return true;
    }
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    hipLaunchKernelGGL((group_norm_forward_rows_any<T, TPR, VPT>),                              \
                       dim3(row_grid(rows, Tile::kRowsPerBlock)), dim3(Tile::kThreads), 0,      \
                       stream, rows, static_cast<int>(L), sh.G, sh.D, sh.S, A(eps),             \
                       static_cast<const T*>(x), static_cast<const A*>(gamma),                  \
                       static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig), \
                       static_cast<T*>(y));                                                     \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
    return true;
  }
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    const unsigned one_shot = row_grid(rows, Tile::kRowsPerBlock);                              \
    note_flavour(sh.S % kVec == 0 ? "group_norm_forward_rows<" #TPR "," #VPT ",0>"           \
                 : sh.S >= kWaveSize * kVec && !(kVec == 8 && VPT == 8 && TPR == 1024)          \
                     ? "group_norm_forward_rows<" #TPR "," #VPT ",2>"                          \
                     : "group_norm_forward_rows<" #TPR "," #VPT ",1>");                        \
    auto kernel = sh.S % kVec == 0 ? group_norm_forward_rows<T, TPR, VPT, 0>                    \
        : sh.S >= kWaveSize * kVec && !(kVec == 8 && VPT == 8 && TPR == 1024) /* spills: 82 us against 66 */ \
            ? group_norm_forward_rows<T, TPR, VPT, 2>                                           \
            : group_norm_forward_rows<T, TPR, VPT, 1>;                                          \
    const unsigned resident = TPR == 1024 ? resident_grid(kernel, TPR, 0) : one_shot;           \
    hipLaunchKernelGGL(kernel,                                                                  \
                       dim3(one_shot < resident ? one_shot : resident), dim3(Tile::kThreads), 0, stream, \
                       rows, static_cast<int>(L), sh.G, sh.D, sh.S, A(eps),                     \
                       static_cast<const T*>(x), static_cast<const A*>(gamma),                  \
                       static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig), \
                       static_cast<T*>(y));                                                     \
  }
  DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  return true;
}

// --------------------------------------------------------------------------
// NHWC, fused forward: one 1024-thread workgroup per sample. A sample is S rows
// of C channels; thread (r, cp) holds packet cp of rows r, r + R, r + 2R, ...
// (R = 1024 / (C / kVec) rows at a time), so its channels, their group and
// their gamma / beta are fixed, and a sample of up to 256 KB stays in registers
// between the statistics and the normalisation: x is read once. A group's sums
// are formed in a fixed order: every thread leaves its partial in LDS, one
// thread per group adds the R * (D / kVec) partials of its group.
// Requires D % kVec == 0 (a packet lies in one group) and C / kVec <= 1024.
// --------------------------------------------------------------------------
constexpr int kSampleThreads = 1024;

// kTwo: D is not a multiple of kVec (but at least kVec): a packet may lie in two
// groups; the thread then carries a share for each, and the elements pick their
// group's statistics one by one.
template <typename T, int kVPT, bool kTwo>
__global__ __launch_bounds__(kSampleThreads) void group_norm_nhwc_samples(
    const uint32_t N, const uint32_t S, const uint32_t C, const uint32_t G, const uint32_t D,
    const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  __shared__ A part[kTwo ? 2 : 1][kSampleThreads];
  __shared__ A total[kSampleThreads];  // one word per group (G <= C / kVec <= 1024)
  const uint32_t cps = C / kVec;                     // packets per row
  const uint32_t rows_at_a_time = kSampleThreads / cps;
  const uint32_t t = threadIdx.x;
  const uint32_t r = t / cps, cp = t - r * cps;
  const bool on = r < rows_at_a_time;
  // the group of the packet's first channel, and how many of its channels lie in it
  const uint32_t g = on ? cp * kVec / D : 0u;
  const int k0 = kTwo ? static_cast<int>(min(static_cast<uint32_t>(kVec), (g + 1) * D - cp * kVec)) : kVec;
  const uint32_t g1 = g + 1 < G ? g + 1 : g;
  const A inv_l = A(1) / A(static_cast<int64_t>(D) * S);
  // The groups' totals of one value per thread and share, the same bits in every
  // thread: the thread that owns group t adds the shares of the packets that
  // touch it, row by row.
  auto group_sums = [&](A v0, A v1, A& t0, A& t1) {
    part[0][t] = on ? v0 : A(0);
    if constexpr (kTwo) part[1][t] = on ? v1 : A(0);
    __syncthreads();
    if (t < G) {
      const uint32_t lo = t * D / kVec, hi = ((t + 1) * D - 1) / kVec;
      A acc = A(0);
      for (uint32_t rr = 0; rr < rows_at_a_time; ++rr) {
        for (uint32_t c = lo; c <= hi; ++c) {
          // packet c starts in this group, or (only c == lo) in the one before it
          const int share = kTwo && c * kVec < t * D ? 1 : 0;
          acc += part[share][rr * cps + c];
        }
      }
      total[t] = acc;
    }
    __syncthreads();
    t0 = total[g];
    t1 = kTwo ? total[g1] : A(0);
    __syncthreads();  // (total is rewritten by the next call)
  };

  // (Requesting the next sample's packets inside the store loop, as the backward does, was
  // measured slower here: bf16 [1024, 16*16, 256] 63 -> 66 us, [2048, 14*14, 256] 101 -> 106.)
  for (uint32_t n = blockIdx.x; n < N; n += gridDim.x) {
    const T* xs = x + static_cast<size_t>(n) * S * C;
    T* ys = y + static_cast<size_t>(n) * S * C;
    // element offsets inside a sample fit 32 bits (a sample is at most 256 KB)
    const uint32_t first = r * C + cp * kVec, step = rows_at_a_time * C;
    u32x4 raw[kVPT];
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const bool has = on && r + i * rows_at_a_time < S;
      raw[i] = load_packet(xs + (has ? first + i * step : 0u));
    }
    A s0 = A(0), s1 = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (on && r + i * rows_at_a_time < S) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (!kTwo || e < k0) s0 += v[e]; else s1 += v[e];
        }
      }
    }
    A mean0, mean1;
    group_sums(s0, s1, mean0, mean1);
    mean0 *= inv_l, mean1 *= inv_l;
    // convert the packets again in each pass instead of keeping every converted element
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
    A q0 = A(0), q1 = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (on && r + i * rows_at_a_time < S) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (!kTwo || e < k0) {
            const A d = v[e] - mean0;
            q0 += d * d;
          } else {
            const A d = v[e] - mean1;
            q1 += d * d;
          }
        }
      }
    }
    A rs0, rs1;
    group_sums(q0, q1, rs0, rs1);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
    rs0 = acc_rsqrt_exact(rs0 * inv_l + eps);
    rs1 = kTwo ? acc_rsqrt_exact(rs1 * inv_l + eps) : A(0);
    if (on && r == 0) {
      if (cp * kVec == g * D) {  // the packet opens its first group
        mu[static_cast<size_t>(n) * G + g] = mean0;
        rsig[static_cast<size_t>(n) * G + g] = rs0;
      }
      if (kTwo && k0 < kVec) {  // and its second group starts inside it
        mu[static_cast<size_t>(n) * G + g1] = mean1;
        rsig[static_cast<size_t>(n) * G + g1] = rs1;
      }
    }
    // The thread's channels are the same for every sample, but their parameters
    // are fetched here, per sample, so that they do not occupy registers while
    // the sample is loaded and reduced.
    const A* gp = gamma + (on ? cp * kVec : 0u);
    const A* bp = beta + (on ? cp * kVec : 0u);
    asm volatile("" : "+v"(gp), "+v"(bp));
    A gam[kVec], bet[kVec], mean[kVec];
    load_params_ragged<kVec>(gp, kVec, gam);
    load_params_ragged<kVec>(bp, kVec, bet);
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      const bool head = !kTwo || e < k0;
      gam[e] *= head ? rs0 : rs1;
      mean[e] = head ? mean0 : mean1;
    }
    // (the offsets are formed again rather than kept from the loads: registers)
    uint32_t first_out = first;
    asm volatile("" : "+v"(first_out));
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const uint32_t row = r + i * rows_at_a_time;
      if (on && row < S) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = (v[e] - (kTwo ? mean[e] : mean0)) * gam[e] + bet[e];
        store_packet(ys + (first_out + i * step), IO<T>::pack(v));
      }
    }
  }
}

// true when the kernel above was launched
template <typename T>
bool try_group_norm_forward_nhwc_samples(const GroupShape& sh, float eps, const void* x,
                                         const void* gamma, const void* beta, void* mu, void* rsig,
                                         void* y, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  if constexpr (sizeof(T) > 4) {
    return false;
  } else {
    if (sh.nchw || sh.S <= 1 || sh.C % kVec != 0 || sh.D < static_cast<uint32_t>(kVec) ||
        !aligned16(x) || !aligned16(y)) {
      return false;
    }
    const bool two = sh.D % kVec != 0;  // a packet may lie in two groups
    const uint32_t cps = sh.C / kVec;
    if (cps > kSampleThreads) return false;
    const uint32_t rows_at_a_time = kSampleThreads / cps;
    const int64_t slots = ceil_div(sh.S, rows_at_a_time);
    if (slots > (two ? 8 : 16)) return false;
    // most of the workgroup's threads must have a row to hold
    if (static_cast<int64_t>(cps) * rows_at_a_time * 4 < kSampleThreads * 3) return false;
#define LAUNCH(VPT)                                                                              \
  {                                                                                              \
    note_flavour(two ? "group_norm_nhwc_samples<" #VPT ",two>" : "group_norm_nhwc_samples<" #VPT ">"); \
    auto kernel = two ? group_norm_nhwc_samples<T, VPT < 16 ? VPT : 8, true>                     \
                      : group_norm_nhwc_samples<T, VPT, false>;                                  \
    const unsigned resident = resident_grid(kernel, kSampleThreads, 0);                          \
    hipLaunchKernelGGL(kernel, dim3(sh.N < resident ? sh.N : resident), dim3(kSampleThreads), 0, \
                       stream, sh.N, sh.S, sh.C, sh.G, sh.D, A(eps), static_cast<const T*>(x),   \
                       static_cast<const A*>(gamma), static_cast<const A*>(beta),                \
                       static_cast<A*>(mu), static_cast<A*>(rsig), static_cast<T*>(y));          \
  }
    if (slots <= 4) LAUNCH(4) else if (slots <= 8) LAUNCH(8) else LAUNCH(16)
#undef LAUNCH
    return true;
  }
}

// The backward the same way: x and dy of a sample in registers (up to eight
// packets per thread each, samples of up to 128 KB per tensor), groups of at
// least a packet; kSplitTwo: a group need not be whole packets, so a packet may lie
// in two groups (elements below k0 in group g, the others in g + 1) and a thread
// carries a share for each; kSplitEach: groups narrower than a packet, a share per
// channel of the packet (up to four packets per thread each). ds / db per group
// are added up by a team of threads out of one LDS word per thread and share; a thread's
// channels are the same for every sample it sees, so their dgamma / dbeta
// shares stay in registers across samples and leave the workgroup once, as one
// partial row of 2*C interleaved words per workgroup (summed by
// sum_partial_rows). (Keeping the shares in LDS between samples instead, one
// word per thread and share, freed no registers where they are short, in the
// two-group flavour at eight packets per thread, and was not faster.)
constexpr uint32_t kMaxEachGroups = 256;     // groups narrower than a packet: groups and channels
constexpr uint32_t kMaxEachChannels = 1024;  // whose statistics and coefficients fit the LDS tables
template <typename T, int kVPT, int kThreads, int kSplit>
__global__ __launch_bounds__(kThreads, 4) void group_norm_grad_nhwc_samples(
    const uint32_t N, const uint32_t S, const uint32_t C, const uint32_t G, const uint32_t D,
    const T* __restrict__ x, const T* __restrict__ dy, const typename IO<T>::Acc* __restrict__ gamma,
    const typename IO<T>::Acc* __restrict__ mu, const typename IO<T>::Acc* __restrict__ rsig,
    typename IO<T>::Acc* __restrict__ ds, typename IO<T>::Acc* __restrict__ db, T* __restrict__ dx,
    typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr bool kTwo = kSplit == kSplitTwo, kEach = kSplit == kSplitEach;
  __shared__ A part[kEach ? kVec : kTwo ? 4 : 2][kThreads];
  __shared__ A total[2][kThreads];
  // kEach: the sample's mu / rsig per group, and the three coefficients of dx per channel. They
  // wait in LDS, not in registers: what does not fit the registers is spilled to memory, and a
  // reload inside the store loop queues behind the packets requested ahead.
  __shared__ A stat[2][kEach ? kMaxEachGroups : 1];
  __shared__ A coef[3][kEach ? kMaxEachChannels : 1];
  const uint32_t cps = C / kVec;
  const uint32_t rows_at_a_time = kThreads / cps;
  const uint32_t t = threadIdx.x;
  const uint32_t r = t / cps, cp = t - r * cps;
  const bool on = r < rows_at_a_time;
  const uint32_t lanes_per_group = D / kVec;  // (whole packets only)
  const uint32_t team = team_size(G, rows_at_a_time, kThreads);
  uint32_t g, g1 = 0;
  int k0 = kVec;
  if constexpr (kSplit != kSplitNone) {
    g = on ? cp * kVec / D : 0u;
    const uint32_t edge = (g + 1) * D - (on ? cp : 0u) * kVec;  // >= 1
    if (on && edge < static_cast<uint32_t>(kVec)) k0 = static_cast<int>(edge);
    g1 = k0 < kVec ? g + 1 : g;
  } else {
    g = on ? cp / lanes_per_group : 0u;
  }
  const A denom = A(1) / A(static_cast<int64_t>(D) * S);
  A gam[kVec];
  load_params_ragged<kVec>(gamma + (on ? cp * kVec : 0u), kVec, gam);
  A t1[kVec], t2[kVec];
#pragma unroll
  for (int e = 0; e < kVec; ++e) t1[e] = t2[e] = A(0);

  const uint32_t first = r * C + cp * kVec, step = rows_at_a_time * C;
  // The next sample's packets are requested while this one's dx is stored.
  u32x4 rx[kVPT], rd[kVPT];
  if (blockIdx.x < N) {
    const size_t base = static_cast<size_t>(blockIdx.x) * S * C;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const bool has = on && r + i * rows_at_a_time < S;
      rx[i] = load_packet(x + base + (has ? first + i * step : 0u));
      rd[i] = load_packet(dy + base + (has ? first + i * step : 0u));
    }
  }
  for (uint32_t n = blockIdx.x; n < N; n += gridDim.x) {
    const size_t base = static_cast<size_t>(n) * S * C;
    const bool more = n + gridDim.x < N;  // uniform over the workgroup
    const size_t nbase = static_cast<size_t>(more ? n + gridDim.x : n) * S * C;
    A m = A(0), rs = A(0), mb = A(0), rsb = A(0), u0 = A(0), v0 = A(0), u0b = A(0), v0b = A(0);
    if constexpr (kEach) {
      if (t < G) {  // requested now, used after the sums
        stat[0][t] = mu[static_cast<size_t>(n) * G + t];
        stat[1][t] = rsig[static_cast<size_t>(n) * G + t];
      }
      // Groups narrower than a packet: every channel of the packet finds its own group. A
      // channel's sums of dy x and dy over the thread's rows give its share of the group's ds /
      // db (times gamma) and of dgamma / dbeta ((sum(dy x) - mu sum(dy)) rsig, as the CPU
      // kernel forms them per (n, c)).
      A a[kVec], b[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) a[e] = b[e] = A(0);
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        // (one packet at a time: converted all at once they would not fit the registers)
        asm volatile("" : "+v"(rx[i]), "+v"(rd[i]), "+v"(a[0]), "+v"(b[0]));
        if (on && r + i * rows_at_a_time < S) {
          A xv[kVec], dv[kVec];
          IO<T>::unpack(rx[i], xv);
          IO<T>::unpack(rd[i], dv);
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            a[e] += dv[e] * xv[e];
            b[e] += dv[e];
          }
        }
      }
      auto channels_of_group = [&](uint32_t gg, uint32_t rr, A (&acc)[1]) {
        for (uint32_t ch = gg * D; ch < (gg + 1) * D; ++ch) {
          acc[0] += part[ch % kVec][rr * cps + ch / kVec];
        }
      };
#pragma unroll
      for (int e = 0; e < kVec; ++e) part[e][t] = on ? gam[e] * a[e] : A(0);
      __syncthreads();
      team_sums<1, A>(G, rows_at_a_time, team, total, channels_of_group);
#pragma unroll
      for (int e = 0; e < kVec; ++e) part[e][t] = on ? gam[e] * b[e] : A(0);
      __syncthreads();
      team_sums<1, A>(G, rows_at_a_time, team, total + 1, channels_of_group);
      if (t < G) {
        ds[static_cast<size_t>(n) * G + t] = total[0][t];
        db[static_cast<size_t>(n) * G + t] = total[1][t];
      }
      // dx = c1 dy + (c2 x + c3) with coefficients per channel: the threads of the first row
      // leave them in LDS for everybody
      uint32_t gc = g, rem = (on ? cp : 0u) * kVec - g * D;  // rem < D
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (rem >= D) rem -= D, ++gc;
        const uint32_t ge = gc < G ? gc : G - 1;
        ++rem;
        const A me = stat[0][ge], re = stat[1][ge];
        if (t < cps) {
          const A q1 = total[0][ge], q2 = total[1][ge];
          const A u = (q2 * me - q1) * (re * re * re) * denom;
          coef[0][t * kVec + e] = gam[e] * re;
          coef[1][t * kVec + e] = u;
          coef[2][t * kVec + e] = -(u * me + q2 * re * denom);
        }
        t1[e] += (a[e] - me * b[e]) * re;
        t2[e] += b[e];
      }
      __syncthreads();
    } else {
      m = mu[static_cast<size_t>(n) * G + g], rs = rsig[static_cast<size_t>(n) * G + g];
      mb = kTwo ? mu[static_cast<size_t>(n) * G + g1] : A(0);
      rsb = kTwo ? rsig[static_cast<size_t>(n) * G + g1] : A(0);
      A s1 = A(0), s2 = A(0), s1b = A(0), s2b = A(0);
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (on && r + i * rows_at_a_time < S) {
          A xv[kVec], dv[kVec];
          IO<T>::unpack(rx[i], xv);
          IO<T>::unpack(rd[i], dv);
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            const A gd = gam[e] * dv[e];
            if (!kTwo || e < k0) {
              s1 += gd * xv[e];
              s2 += gd;
              t1[e] += dv[e] * (xv[e] - m) * rs;
            } else {
              s1b += gd * xv[e];
              s2b += gd;
              t1[e] += dv[e] * (xv[e] - mb) * rsb;
            }
            t2[e] += dv[e];
          }
        }
      }
      // the group's ds and db: one LDS word per thread, share and sum, added up by the group's
      // team of threads
      part[0][t] = on ? s1 : A(0);
      part[1][t] = on ? s2 : A(0);
      if constexpr (kTwo) {
        part[2][t] = on ? s1b : A(0);
        part[3][t] = on ? s2b : A(0);
      }
      __syncthreads();
      if constexpr (kTwo) {
        // packets lo..hi hold the group's channels; one that begins before the group gives its
        // second share
        team_sums<2, A>(G, rows_at_a_time, team, total, [&](uint32_t gg, uint32_t rr, A (&acc)[2]) {
          const uint32_t lo = gg * D / kVec, hi = ((gg + 1) * D - 1) / kVec;
          for (uint32_t c = lo; c <= hi; ++c) {
            const int share = c * kVec < gg * D ? 2 : 0;
            acc[0] += part[share][rr * cps + c];
            acc[1] += part[share + 1][rr * cps + c];
          }
        });
      } else {
        team_sums<2, A>(G, rows_at_a_time, team, total, [&](uint32_t gg, uint32_t rr, A (&acc)[2]) {
          for (uint32_t k = 0; k < lanes_per_group; ++k) {
            acc[0] += part[0][rr * cps + gg * lanes_per_group + k];
            acc[1] += part[1][rr * cps + gg * lanes_per_group + k];
          }
        });
      }
      if (t < G) {
        ds[static_cast<size_t>(n) * G + t] = total[0][t];
        db[static_cast<size_t>(n) * G + t] = total[1][t];
      }
      s1 = total[0][g], s2 = total[1][g];
      u0 = (s2 * m - s1) * (rs * rs * rs) * denom;
      v0 = s2 * rs * denom;
      if constexpr (kTwo) {
        s1b = total[0][g1], s2b = total[1][g1];
        u0b = (s2b * mb - s1b) * (rsb * rsb * rsb) * denom;
        v0b = s2b * rsb * denom;
      }
    }
#pragma unroll
    for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(rx[i]), "+v"(rd[i]));
    // (the offsets are formed again rather than kept from the loads: registers)
    uint32_t first_out = first;
    asm volatile("" : "+v"(first_out));
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (on && r + i * rows_at_a_time < S) {
        A xv[kVec], dv[kVec];
        IO<T>::unpack(rx[i], xv);
        IO<T>::unpack(rd[i], dv);
        // (read again for every packet: hoisted out of the loop they would be 3 * kVec registers)
        uint32_t ch0 = cp * kVec;
        asm volatile("" : "+v"(ch0));
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if constexpr (kEach) {
            const uint32_t ch = ch0 + e;
            xv[e] = coef[0][ch] * dv[e] + (coef[1][ch] * xv[e] + coef[2][ch]);
          } else if (!kTwo || e < k0) {
            xv[e] = gam[e] * rs * dv[e] + (u0 * (xv[e] - m) - v0);
          } else {
            xv[e] = gam[e] * rsb * dv[e] + (u0b * (xv[e] - mb) - v0b);
          }
        }
        store_packet(dx + base + (first_out + i * step), IO<T>::pack(xv));
      }
      if (more) {
        const bool has = on && r + i * rows_at_a_time < S;
        rx[i] = load_packet(x + nbase + (has ? first_out + i * step : 0u));
        rd[i] = load_packet(dy + nbase + (has ? first_out + i * step : 0u));
      }
    }
    __syncthreads();  // total is rewritten for the next sample
  }
  // this workgroup's partial row: per channel, the shares of its row threads in row order
  A* row = partial + static_cast<size_t>(blockIdx.x) * 2 * C;
  A (*lds)[kThreads] = part;
#pragma unroll
  for (int e = 0; e < kVec; ++e) {
    lds[0][t] = on ? t1[e] : A(0);
    lds[1][t] = on ? t2[e] : A(0);
    __syncthreads();
    if (t < cps) {
      A a = A(0), b = A(0);
      for (uint32_t rr = 0; rr < rows_at_a_time; ++rr) {
        a += lds[0][rr * cps + t];
        b += lds[1][rr * cps + t];
      }
      row[2 * (t * kVec + e)] = a;
      row[2 * (t * kVec + e) + 1] = b;
    }
    __syncthreads();
  }
}

// Workgroup size for a sample: the smallest of 256, 512 and 1024 threads (four, two and one
// workgroup per compute unit; several overlap their phases) whose eight packets per thread and
// tensor hold it; 0: none.
template <typename T>
int group_norm_grad_nhwc_samples_threads(const GroupShape& sh, int* slots_out) {
  constexpr int kVec = IO<T>::kVec;
  if (sizeof(T) > 4 || sh.nchw || sh.S <= 1 || sh.C % kVec != 0) return 0;
  if (sh.G > 256) return 0;  // (a team of threads per group)
  if (sh.D < kVec && sh.C > kMaxEachChannels) return 0;
  const uint32_t cps = sh.C / kVec;
  // Groups narrower than a packet keep a sum of dy x and of dy per channel: four packets per
  // thread and tensor at most (80 bytes per thread are spilled there in 16-bit types, outside
  // the store loop; the smaller workgroup is still ahead of two packets on twice the threads:
  // bf16 [8192,16*16,32] 106 against 119 us). Groups that are not whole packets look for four
  // packets first: at eight the two-group flavour spills 110 bytes per thread, and what it
  // reloads inside the store loop queues behind the packets requested ahead (bf16
  // [1024,8*8,320] 50 us on 512 threads with eight packets, 39 us on 1024 with four). Groups of
  // whole packets are better off with eight packets on the smaller workgroup (76-81 us against
  // 80-90 us on 64 KB samples).
  for (const int64_t most : {sh.D % kVec != 0 ? 4 : 8, sh.D < kVec ? 4 : 8}) {
    for (const uint32_t threads : {256u, 512u, 1024u}) {
      if (cps > threads) continue;
      const uint32_t rows_at_a_time = threads / cps;
      const int64_t slots = ceil_div(sh.S, rows_at_a_time);
      if (slots > most) continue;
      // most of the workgroup's threads must have a row to hold
      if (static_cast<int64_t>(cps) * rows_at_a_time * 4 < threads * 3) continue;
      *slots_out = static_cast<int>(slots);
      return static_cast<int>(threads);
    }
  }
  return 0;
}

template <typename T>
int launch_group_norm(const GroupShape& sh, const void* x, const void* mu, const void* rsig,
                      const void* gamma, const void* beta, void* y, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const uint32_t total = sh.N * sh.C * sh.S;
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  const bool vec_ok = aligned16(x) && aligned16(y) && (sh.nchw ? sh.S % kVec == 0 : sh.C % kVec == 0);
  ShortPlan sp;
  if (short_group_rows(sh, sizeof(T), x, x, y) && plan_short_rows(sh.S, sizeof(T), 4, false, &sp)) {
    // (n, c) rows that are not whole aligned packets: staged through LDS
    const GroupNormApply<T, 1> f{sh, static_cast<const A*>(mu), static_cast<const A*>(rsig),
                                 static_cast<const A*>(gamma), static_cast<const A*>(beta)};
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16 + sp.rows_per_chunk * 4 * sizeof(A);
    DRAGON_HIP_SHORT_LAUNCH(T, GroupRowApply, sp, lds, short_grid(rows, sp.rows_per_chunk), stream,
                            rows, static_cast<int>(sh.S), xp, xp, yp, f);
  } else if (long_group_rows(sh, sizeof(T), x, x, y)) {
    // longer rows of that kind: one wavefront per row
    const GroupRowApply<T, 8> op{GroupNormApply<T, 1>{
        sh, static_cast<const A*>(mu), static_cast<const A*>(rsig), static_cast<const A*>(gamma),
        static_cast<const A*>(beta)}};
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    if constexpr (sizeof(T) <= 4) {
      // the aligned packets that cover the tensor, the row's scalars found once per packet
      hipLaunchKernelGGL((map_flat_windows<T, 1, GroupRowApply<T, 8>>),
                         dim3(map_grid(total / kVec + 2)), dim3(256), 0, stream, total, sh.S, xp, xp,
                         yp, op);
    } else {
      hipLaunchKernelGGL((long_rows_map<T, 1, GroupRowApply<T, 8>>), dim3(long_rows_grid(rows)),
                         dim3(kLongThreads), 0, stream, rows, static_cast<int>(sh.S), xp, xp, yp, op);
    }
  } else if (vec_ok) {
    GroupNormApply<T, kVec> f{sh, static_cast<const A*>(mu), static_cast<const A*>(rsig),
                              static_cast<const A*>(gamma), static_cast<const A*>(beta)};
    hipLaunchKernelGGL((map_flat<T, 1, kVec, GroupNormApply<T, kVec>>), dim3(map_grid(total / kVec)),
                       dim3(256), 0, stream, total, xp, xp, yp, f);
  } else {
    GroupNormApply<T, 1> f{sh, static_cast<const A*>(mu), static_cast<const A*>(rsig),
                           static_cast<const A*>(gamma), static_cast<const A*>(beta)};
    hipLaunchKernelGGL((map_flat<T, 1, 1, GroupNormApply<T, 1>>), dim3(map_grid(total)), dim3(256), 0,
                       stream, total, xp, xp, yp, f);
  }
  return status_of_launch();
}

template <typename T>
int launch_group_norm_grad(const GroupShape& sh, const void* x, const void* mu, const void* rsig,
                           const void* gamma, const void* dy, void* ds, void* db, void* dgamma,
                           void* dbeta, void* dx, void* scratch, size_t scratch_bytes,
                           hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* xp = static_cast<const T*>(x);
  const T* dyp = static_cast<const T*>(dy);
  T* dxp = static_cast<T*>(dx);
  const A* mup = static_cast<const A*>(mu);
  const A* rsp = static_cast<const A*>(rsig);
  const A* gp = static_cast<const A*>(gamma);
  A* dsp = static_cast<A*>(ds);
  A* dbp = static_cast<A*>(db);
  A* dgp = static_cast<A*>(dgamma);
  A* dbtp = static_cast<A*>(dbeta);
  A* part = static_cast<A*>(scratch);
  const int layout = sh.nchw ? DRAGON_HIP_NCHW : DRAGON_HIP_NHWC;
  if (scratch_bytes < group_norm_grad_scratch<T>(sh.N, sh.G, sh.D, sh.S, layout) || !scratch) {
    return DRAGON_HIP_ESCRATCH;
  }

  ShortPlan sp;
  auto ln_lds_of = [](const ShortPlan& q) {
    return static_cast<size_t>(q.stage_packets) * 32 + q.rows_per_chunk * 2 * sizeof(A);
  };
  if (layer_norm_grad_short_rows(sh.G, sh.D, sh.S, sizeof(T), x, dy, dx) &&
      plan_short_rows_within(sh.D, sizeof(T), 4, aligned16(x), ln_lds_of, &sp)) {
    // 16 KB per staged tensor: eight loads in flight per thread while staging
    // ([1048576, 64] bf16 95 -> 80 us against 8 KB)
    size_t lds = ln_lds_of(sp);
    const size_t end_bytes = static_cast<size_t>(kShortThreads) * sp.per_lane * 2 * sizeof(A);
    if (lds < end_bytes) lds = end_bytes;
    const unsigned grid = short_grad_grid(sh.N, sp.rows_per_chunk);
    const int64_t rows = sh.N;
    DRAGON_HIP_SHORT_LAUNCH(T, LayerNormShortBackward, sp, lds, grid, stream, rows,
                            static_cast<int>(sh.D), xp, dyp, dxp, A(1) / A(sh.D), mup, rsp, gp, dsp,
                            dbp, part, {}, {}, {});
    launch_sum_partial_rows<A>(grid, sh.D, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  const RowGradPlan rp = plan_row_grad<T>(sh.N, sh.G, sh.D, sh.S);
  if (rp.use_rows) {
    // rows of whole aligned packets, or the ragged flavour for any width and alignment
    const bool ragged =
        rp.ragged || !(aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(gamma));
    const size_t staged_bytes = static_cast<size_t>(ceil_div(sh.D, kVec) * kVec) * sizeof(A);
    const TimelineTarget& tl = timeline_target();
    unsigned long long* marks = tl.stamps != nullptr && tl.workgroups >= rp.grid ? tl.stamps : nullptr;
#define LAUNCH_T(TPR, VPT, THREADS)                                                           \
  {                                                                                           \
    note_flavour(ragged ? "layer_norm_grad_rows<" #TPR "," #VPT "," #THREADS ",ragged>"        \
                        : "layer_norm_grad_rows<" #TPR "," #VPT "," #THREADS ">");             \
    auto kernel = ragged ? layer_norm_grad_rows<T, TPR, VPT, THREADS, true>                   \
                         : layer_norm_grad_rows<T, TPR, VPT, THREADS, false>;                 \
    if (staged_bytes > 48 * 1024) (void)resident_grid(kernel, THREADS, staged_bytes);         \
    hipLaunchKernelGGL(kernel, dim3(rp.grid), dim3(THREADS), staged_bytes, stream,            \
                       static_cast<int64_t>(sh.N), static_cast<int>(sh.D), xp, dyp, gp, mup,  \
                       rsp, dsp, dbp, dxp, part, marks);                                      \
  }
#define LAUNCH(TPR, VPT)                                                    \
  {                                                                         \
    if constexpr (VPT * IO<T>::kVec <= 16 || sizeof(A) == 8) {              \
      if constexpr (TPR >= 768) {                                           \
        LAUNCH_T(TPR, VPT, TPR)                                             \
      } else {                                                              \
        LAUNCH_T(TPR, VPT, 512)                                             \
      }                                                                     \
    }                                                                       \
  }
    if (rp.cfg.tpr == 64 && rp.cfg.vpt == 1) LAUNCH(64, 1)
    else if (rp.cfg.tpr == 64 && rp.cfg.vpt == 2) LAUNCH(64, 2)
    else if (rp.cfg.tpr == 256 && rp.cfg.vpt == 1) LAUNCH(256, 1)
    else if (rp.cfg.tpr == 256 && rp.cfg.vpt == 2 && rp.threads == 1024) {
      if constexpr (IO<T>::kVec == 8) LAUNCH_T(256, 2, 1024)
    }
    else if (rp.cfg.tpr == 256 && rp.cfg.vpt == 2) LAUNCH(256, 2)
    else if (rp.cfg.tpr == 512 && rp.cfg.vpt == 2 && rp.threads == 1024) {
      if constexpr (IO<T>::kVec < 8) LAUNCH_T(512, 2, 1024)
    }
    else if (rp.cfg.tpr == 512 && rp.cfg.vpt == 1) LAUNCH(512, 1)
    else if (rp.cfg.tpr == 512 && rp.cfg.vpt == 2) LAUNCH(512, 2)
    else if (rp.cfg.tpr == 1024 && rp.cfg.vpt == 1) LAUNCH(1024, 1)
    else if (rp.cfg.tpr == 768 && rp.cfg.vpt == 2) LAUNCH(768, 2)
    else if (rp.cfg.tpr == 1024 && rp.cfg.vpt == 2) LAUNCH(1024, 2)
    else LAUNCH(1024, 4)
#undef LAUNCH_T
#undef LAUNCH
    launch_sum_partial_rows<A>(rp.grid, sh.D, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  if (sh.G == 1 && sh.S == 1) {
    // rows beyond the register tiles: row sums, then dx with column partials
    const bool packets = sh.D % kVec == 0 && aligned16(x) && aligned16(dy) && aligned16(dx) &&
        aligned16(gamma);
    const WideGradPlan wp = plan_wide_grad(sh.N, sh.D, packets ? kVec : 1);
    A* pairs = part;
    A* rows = part + wide_grad_pair_words(sh.N, wp);
    const dim3 first(sh.N * wp.splits), second(wp.col_blocks * wp.row_chunks);
    const int D = static_cast<int>(sh.D);
    if (packets) {
      hipLaunchKernelGGL((layer_norm_wide_row_sums<T, kVec>), first, dim3(kReduceThreads), 0,
                         stream, D, wp, xp, dyp, gp, pairs);
      hipLaunchKernelGGL((layer_norm_wide_grad<T, kVec>), second, dim3(kReduceThreads), 0, stream,
                         static_cast<int64_t>(sh.N), D, wp, xp, dyp, gp, mup, rsp, pairs, dsp, dbp,
                         dxp, rows);
    } else {
      hipLaunchKernelGGL((layer_norm_wide_row_sums<T, 1>), first, dim3(kReduceThreads), 0, stream,
                         D, wp, xp, dyp, gp, pairs);
      hipLaunchKernelGGL((layer_norm_wide_grad<T, 1>), second, dim3(kReduceThreads), 0, stream,
                         static_cast<int64_t>(sh.N), D, wp, xp, dyp, gp, mup, rsp, pairs, dsp, dbp,
                         dxp, rows);
    }
    launch_sum_partial_rows<A>(wp.row_chunks, sh.D, rows, dgp, dbtp, stream);
    return status_of_launch();
  }

  if (ShortPlan gsp; sh.nchw && sh.G * sh.D > 1 && sh.D <= 8 && sizeof(T) <= 4 &&
                     ceil_div(static_cast<int64_t>(sh.D) * sh.S, kVec) <= 32 &&
                     static_cast<int64_t>(sh.N) * sh.G >= 4096 && congruent16(x, dy) &&
                     congruent16(x, dx) &&
                     plan_short_rows_within(
                         static_cast<int64_t>(sh.D) * sh.S, sizeof(T), 3, aligned16(x),
                         [](const ShortPlan& q) { return static_cast<size_t>(q.stage_packets) * 32; },
                         &gsp)) {
    // thousands of groups of at most 32 packets: several groups per wavefront, staged through LDS
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
    const int L = static_cast<int>(sh.D * sh.S);
    const size_t lds = static_cast<size_t>(gsp.stage_packets) * 32;
    DRAGON_HIP_SHORT_LAUNCH(T, GroupShortBackward, gsp, lds, short_grid(rows, gsp.rows_per_chunk),
                            stream, rows, L, xp, dyp, dxp, A(1) / A(L), gp, mup, rsp, dsp, dbp, part,
                            sh.G, sh.D, sh.S, {});
    launch_sum_partial_rows<A>(sh.N, sh.C, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  if (sh.nchw && sh.G * sh.D > 1 && sh.S >= static_cast<uint32_t>(kVec) && (sh.D * sh.S) % kVec == 0 &&
      sh.D * sh.S / kVec <= 4 * kWaveSize && sizeof(T) <= 4 && aligned16(x) && aligned16(dy) &&
      aligned16(dx)) {
    // small groups: a wavefront each
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
    const int L = static_cast<int>(sh.D * sh.S);
    const int64_t want = ceil_div(rows, kWaveGroupThreads / kWaveSize);
    const int64_t cap = static_cast<int64_t>(num_cus()) * 32;
    const dim3 grid(static_cast<unsigned>(want < cap ? want : cap));
    const int packets = L / kVec;
#define LAUNCH(VPT)                                                                             \
  hipLaunchKernelGGL((group_norm_grad_wave_groups<T, VPT>), grid, dim3(kWaveGroupThreads), 0,   \
                     stream, rows, L, sh.G, sh.D, sh.S, xp, dyp, gp, mup, rsp, dsp, dbp, dxp, part);
    if (packets <= kWaveSize) LAUNCH(1) else if (packets <= 2 * kWaveSize) LAUNCH(2) else LAUNCH(4)
#undef LAUNCH
    launch_sum_partial_rows<A>(sh.N, sh.C, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  if (const int64_t wp = static_cast<int64_t>(sh.D) * sh.S / kVec + 2;
      sh.nchw && sh.G * sh.D > 1 && sizeof(T) <= 4 && sh.S >= static_cast<uint32_t>(kVec) &&
      ((sh.D * sh.S) % kVec != 0 || !aligned16(x)) && congruent16(x, dy) && congruent16(x, dx) &&
      wp > 2 * kWaveSize && wp <= kMaxEntryPackets) {
    // groups that are not whole aligned packets themselves: through their packet windows
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
    const int L = static_cast<int>(sh.D * sh.S);
    const unsigned grid = static_cast<unsigned>(rows < (1 << 20) ? rows : (1 << 20));
    const size_t lds = static_cast<size_t>(wp) * 4 * sizeof(A);
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    note_flavour("group_norm_grad_rows_any<" #TPR "," #VPT ",window>");                         \
    auto kernel = group_norm_grad_rows_any<T, TPR, VPT, true>;                                  \
    if (lds > 32 * 1024) (void)resident_grid(kernel, TPR, lds);                                 \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(TPR), lds, stream, rows, L, sh.G, sh.D, sh.S,   \
                       xp, dyp, gp, mup, rsp, dsp, dbp, dxp, part);                             \
  }
    if (wp <= 256 * 2) LAUNCH(256, 2)
    else if (wp <= 256 * 4) LAUNCH(256, 4)
    else if (wp <= 256 * 8) LAUNCH(256, 8)
    else LAUNCH(1024, 4)
#undef LAUNCH
    launch_sum_partial_rows<A>(sh.N, sh.C, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  RowConfig gcfg;
  int mode = kChannelWaves;
  if (plan_group_grad_rows<T>(sh.G, sh.D, sh.S, layout, &gcfg, &mode) && aligned16(x) &&
      aligned16(dy) && aligned16(dx)) {
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
    const int L = static_cast<int>(sh.D * sh.S);
    const unsigned grid = static_cast<unsigned>(rows < (1 << 20) ? rows : (1 << 20));
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
  if (mode == kChannelPackets) {                                                                \
    if constexpr (TPR * VPT <= kMaxEntryPackets && TPR != 512) {                                \
      note_flavour("group_norm_grad_rows_any<" #TPR "," #VPT ">");                              \
      auto kernel = group_norm_grad_rows_any<T, TPR, VPT>;                                      \
      const size_t lds = static_cast<size_t>(L / kVec) * 4 * sizeof(A);                         \
      if (lds > 32 * 1024) (void)resident_grid(kernel, TPR, lds);                               \
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(TPR), lds, stream, rows, L, sh.G, sh.D, sh.S, \
                         xp, dyp, gp, mup, rsp, dsp, dbp, dxp, part);                           \
    }                                                                                           \
  } else {                                                                                      \
    note_flavour(mode == kChannelStraddles ? "group_norm_grad_rows<" #TPR "," #VPT ",straddles>"  \
                 : mode == kChannelStraddlesAny ? "group_norm_grad_rows<" #TPR "," #VPT ",straddles_any>" \
                 : mode == kChannelLanes ? "group_norm_grad_rows<" #TPR "," #VPT ",lanes>"      \
                                         : "group_norm_grad_rows<" #TPR "," #VPT ",waves>");     \
    auto kernel = mode == kChannelStraddles ? group_norm_grad_rows<T, TPR, VPT, kChannelStraddles> \
        : mode == kChannelStraddlesAny ? group_norm_grad_rows<T, TPR, VPT, kChannelStraddlesAny>   \
        : mode == kChannelLanes             ? group_norm_grad_rows<T, TPR, VPT, kChannelLanes>     \
                                            : group_norm_grad_rows<T, TPR, VPT, kChannelWaves>;    \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(TPR), 0, stream, rows, L, sh.G, sh.D, sh.S, xp, \
                       dyp, gp, mup, rsp, dsp, dbp, dxp, part);                                 \
  }                                                                                             \
  }
    if (gcfg.tpr == 256 && gcfg.vpt == 2) LAUNCH(256, 2)
    else if (gcfg.tpr == 256 && gcfg.vpt == 4) LAUNCH(256, 4)
    else if (gcfg.tpr == 256 && gcfg.vpt == 8) LAUNCH(256, 8)
    else if (gcfg.tpr == 512 && gcfg.vpt == 8) LAUNCH(512, 8)
    else if (gcfg.tpr == 1024 && gcfg.vpt == 4) LAUNCH(1024, 4)
    else LAUNCH(1024, 8)
#undef LAUNCH
    launch_sum_partial_rows<A>(sh.N, sh.C, part, dgp, dbtp, stream);
    return status_of_launch();
  }

  {
    const int st = try_group_norm_grad_slices<T>(sh, x, mu, rsig, gamma, dy, ds, db, dgamma, dbeta,
                                                 dx, scratch, stream);
    if (st != kNotApplicable) return st;
  }

  if constexpr (sizeof(T) <= 4) {
    int slots = 0;
    const int threads = group_norm_grad_nhwc_samples_threads<T>(sh, &slots);
    if (threads != 0 && aligned16(x) && aligned16(dy) && aligned16(dx)) {
      // NHWC samples that fit one workgroup's registers: x and dy read once
      unsigned grid = 0;
#define LAUNCH(VPT, THREADS)                                                                     \
  {                                                                                              \
    /* how a packet's channels lie in groups */                                                  \
    const int split = sh.D % kVec == 0 ? kSplitNone : sh.D > kVec ? kSplitTwo : kSplitEach;      \
    note_flavour(split == kSplitEach ? "group_norm_grad_nhwc_samples<" #VPT "," #THREADS ",each>" \
                 : split == kSplitTwo ? "group_norm_grad_nhwc_samples<" #VPT "," #THREADS ",two>" \
                                      : "group_norm_grad_nhwc_samples<" #VPT "," #THREADS ">");  \
    auto kernel = split == kSplitTwo ? group_norm_grad_nhwc_samples<T, VPT, THREADS, kSplitTwo>  \
                                     : group_norm_grad_nhwc_samples<T, VPT, THREADS, kSplitNone>; \
    if constexpr (VPT <= 4) { /* (narrow groups never take eight packets per thread) */          \
      if (split == kSplitEach) kernel = group_norm_grad_nhwc_samples<T, VPT, THREADS, kSplitEach>; \
    }                                                                                            \
    const unsigned resident = resident_grid(kernel, THREADS, 0);                                 \
    grid = nhwc_sample_rows(sh.N);                                                               \
    if (grid > resident) grid = resident;                                                        \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), 0, stream, sh.N, sh.S, sh.C, sh.G,     \
                       sh.D, xp, dyp, gp, mup, rsp, dsp, dbp, dxp, part);                        \
  }
      if (threads == 256) {
        if (slots <= 2) LAUNCH(2, 256) else if (slots <= 4) LAUNCH(4, 256) else LAUNCH(8, 256)
      } else if (threads == 512) {
        // (with groups of a packet or more, a sample of four packets per thread or fewer fits
        // 256 threads; narrower groups look for two packets per thread first)
        if (slots <= 4 && sh.D < static_cast<uint32_t>(kVec)) {
#define LAUNCH_EACH(VPT)                                                                         \
  {                                                                                              \
    note_flavour("group_norm_grad_nhwc_samples<" #VPT ",512,each>");                             \
    auto kernel = group_norm_grad_nhwc_samples<T, VPT, 512, kSplitEach>;                         \
    const unsigned resident = resident_grid(kernel, 512, 0);                                     \
    grid = nhwc_sample_rows(sh.N);                                                               \
    if (grid > resident) grid = resident;                                                        \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), 0, stream, sh.N, sh.S, sh.C, sh.G, sh.D,   \
                       xp, dyp, gp, mup, rsp, dsp, dbp, dxp, part);                              \
  }
          if (slots <= 2) LAUNCH_EACH(2) else LAUNCH_EACH(4)
#undef LAUNCH_EACH
        } else {
          LAUNCH(8, 512)
        }
      } else {
        if (slots <= 2) LAUNCH(2, 1024) else if (slots <= 4) LAUNCH(4, 1024) else LAUNCH(8, 1024)
      }
#undef LAUNCH
      launch_sum_partial_rows<A>(grid, sh.C, part, dgp, dbtp, stream);
      return status_of_launch();
    }
  }

  const uint32_t total = sh.N * sh.C * sh.S;
  const bool base_ok = aligned16(x) && aligned16(dy) && aligned16(dx);
  if (sh.nchw) {
    // 1+2. one pass over x and dy for the per-(n, c) pairs, then ds/db and dgamma/dbeta from them
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    RowConfig cfg;
    ShortPlan sp;
    auto sums_lds_of = [](const ShortPlan& q) {
      return static_cast<size_t>(q.stage_packets) * 32 + q.rows_per_chunk * sizeof(A);
    };
    if (short_group_rows(sh, sizeof(T), x, dy, dx) &&
        plan_short_rows_within(sh.S, sizeof(T), 3, false, sums_lds_of, &sp)) {
      const size_t lds = sums_lds_of(sp);
      T* none = nullptr;
      DRAGON_HIP_SHORT_LAUNCH(T, GroupRowPairSums, sp, lds, short_grid(rows, sp.rows_per_chunk),
                              stream, rows, static_cast<int>(sh.S), xp, dyp, none, mup, sh.D, part);
    } else if (const uint32_t split = few_long_rows_split(rows, sh.S);
               split > 0 && sizeof(T) <= 4 && long_group_rows(sh, sizeof(T), x, dy, dx)) {
      const SegmentedReduce s{static_cast<uint32_t>(rows), 1u, sh.S, 0u, 1u, sh.S, 0u, split};
      A* partial = part + static_cast<size_t>(rows) * 2;
      hipLaunchKernelGGL((reduce2_segments_windows<T, 2, RowPairAccum<T>>), dim3(s.n_out * s.split),
                         dim3(kReduceThreads), 0, stream, s, xp, dyp, RowPairAccum<T>{mup, sh.D, A(0)},
                         partial);
      hipLaunchKernelGGL((reduce2_finalize<A, StorePairs<A>>),
                         dim3(static_cast<unsigned>(ceil_div(rows, kReduceThreads))),
                         dim3(kReduceThreads), 0, stream, s.n_out, s.split, true, partial,
                         StorePairs<A>{part});
    } else if (long_group_rows(sh, sizeof(T), x, dy, dx)) {
      const GroupRowPairSums<T, 8> op{mup, sh.D, part};
      hipLaunchKernelGGL((long_rows_sums<T, 2, GroupRowPairSums<T, 8>>), dim3(long_rows_grid(rows)),
                         dim3(kLongThreads), 0, stream, rows, static_cast<int>(sh.S), xp, dyp, op,
                         part);
    } else if (sh.S < 16) {
      hipLaunchKernelGGL((channel_pair_sums_short<T>), dim3(map_grid(static_cast<uint32_t>(rows))),
                         dim3(256), 0, stream, rows, static_cast<int>(sh.S), sh.D, xp, dyp, mup,
                         part);
    } else if (pick_row_config(ceil_div(sh.S, kVec), 4, &cfg)) {
      const bool regular = sh.S % kVec == 0 && aligned16(x) && aligned16(dy);
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    const dim3 grid(row_grid(rows, Tile::kRowsPerBlock)), block(Tile::kThreads);                \
    if (regular) {                                                                              \
      hipLaunchKernelGGL((channel_pair_sums_rows<T, TPR, VPT, false>), grid, block, 0, stream,  \
                         rows, static_cast<int>(sh.S), sh.D, xp, dyp, mup, part);               \
    } else {                                                                                    \
      hipLaunchKernelGGL((channel_pair_sums_rows<T, TPR, VPT, true>), grid, block, 0, stream,   \
                         rows, static_cast<int>(sh.S), sh.D, xp, dyp, mup, part);               \
    }                                                                                           \
  }
      DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
    } else {
      hipLaunchKernelGGL((channel_pair_sums_looped<T>), dim3(loop_grid(rows)), dim3(kLoopThreads),
                         0, stream, rows, static_cast<int64_t>(sh.S), sh.D, xp, dyp, mup, part);
    }
    const uint32_t group_blocks = group_sum_blocks(sh);
    const uint32_t chan_blocks = static_cast<uint32_t>(ceil_div(sh.C, kWaveSize));
    hipLaunchKernelGGL((group_grad_from_channel_sums<A>), dim3(group_blocks + chan_blocks),
                       dim3(256), 0, stream, sh.N, sh.G, sh.D, group_blocks, part, gp, mup, rsp,
                       dsp, dbp, dgp, dbtp);
  } else {
    // NHWC: the same per-(n, c) pairs from full-width column reductions of each sample
    A* sums = part + batched_partial_pairs(sh.N, sh.S, sh.C) * 2;
    const BatchedColumns d = launch_batched_columns<T, 2>(
        sh, xp, dyp, ColumnPairAccum<T>{mup, sh.G, sh.D, A(0)}, part, stream);
    hipLaunchKernelGGL((sum_batched_partials<A>),
                       dim3(static_cast<unsigned>(ceil_div(sh.N * sh.C, 256))), dim3(256), 0,
                       stream, d, part, sums);
    const uint32_t group_blocks = group_sum_blocks(sh);
    const uint32_t chan_blocks = static_cast<uint32_t>(ceil_div(sh.C, kWaveSize));
    hipLaunchKernelGGL((group_grad_from_channel_sums<A>), dim3(group_blocks + chan_blocks),
                       dim3(256), 0, stream, sh.N, sh.G, sh.D, group_blocks, sums, gp, mup, rsp,
                       dsp, dbp, dgp, dbtp);
  }
  // 3. dx
  {
    const A denom = A(1) / A(static_cast<int64_t>(sh.D) * sh.S);
    const bool vec_ok = base_ok && (sh.nchw ? sh.S % kVec == 0 : sh.C % kVec == 0);
    ShortPlan sp;
    auto map_lds_of = [](const ShortPlan& q) {
      return static_cast<size_t>(q.stage_packets) * 32 + q.rows_per_chunk * 6 * sizeof(A);
    };
    if (short_group_rows(sh, sizeof(T), x, dy, dx) &&
        plan_short_rows_within(sh.S, sizeof(T), 3, false, map_lds_of, &sp)) {
      const GroupNormGradApply<T, 1> f{sh, mup, rsp, gp, dsp, dbp, denom};
      const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
      const size_t lds = map_lds_of(sp);
      DRAGON_HIP_SHORT_LAUNCH(T, GroupRowGradMap, sp, lds, short_grid(rows, sp.rows_per_chunk),
                              stream, rows, static_cast<int>(sh.S), xp, dyp, dxp, f);
    } else if (long_group_rows(sh, sizeof(T), x, dy, dx)) {
      const GroupRowGradMap<T, 8> op{GroupNormGradApply<T, 1>{sh, mup, rsp, gp, dsp, dbp, denom}};
      const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
      if constexpr (sizeof(T) <= 4) {
        hipLaunchKernelGGL((map_flat_windows<T, 2, GroupRowGradMap<T, 8>>),
                           dim3(map_grid(total / kVec + 2)), dim3(256), 0, stream, total, sh.S, xp,
                           dyp, dxp, op);
      } else {
        hipLaunchKernelGGL((long_rows_map<T, 2, GroupRowGradMap<T, 8>>), dim3(long_rows_grid(rows)),
                           dim3(kLongThreads), 0, stream, rows, static_cast<int>(sh.S), xp, dyp, dxp,
                           op);
      }
    } else if (vec_ok) {
      GroupNormGradApply<T, kVec> f{sh, mup, rsp, gp, dsp, dbp, denom};
      hipLaunchKernelGGL((map_flat<T, 2, kVec, GroupNormGradApply<T, kVec>>),
                         dim3(map_grid(total / kVec)), dim3(256), 0, stream, total, xp, dyp, dxp, f);
    } else {
      GroupNormGradApply<T, 1> f{sh, mup, rsp, gp, dsp, dbp, denom};
      hipLaunchKernelGGL((map_flat<T, 2, 1, GroupNormGradApply<T, 1>>), dim3(map_grid(total)),
                         dim3(256), 0, stream, total, xp, dyp, dxp, f);
    }
  }
  return status_of_launch();
}

// NHWC statistics of the fused forward: column sums per sample, then mean and
// rsig per group (InvStd folded into the second stage).
// Statistics of NCHW groups whose rows of D*S elements are not whole aligned
// packets and exceed the register tiles: one wavefront per group row, then
// mean and rsig from the shifted sums. kNotApplicable leaves the call to Moments.
template <typename T>
int try_group_norm_stats_rows(const GroupShape& sh, float eps, const void* x, void* mu, void* rsig,
                              void* scratch, size_t scratch_bytes, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const int64_t L = static_cast<int64_t>(sh.D) * sh.S;
  const int64_t rows = static_cast<int64_t>(sh.N) * sh.G;
  const bool packets = L % kVec == 0 && aligned16(x);
  if (!sh.nchw || packets || L <= 1024 || !fits_int32(L)) return kNotApplicable;
  // fewer rows than that are too few wavefronts: Moments splits each row over several workgroups
  if (rows < 2048 && sizeof(T) <= 4) return kNotApplicable;
  if (!scratch || scratch_bytes < static_cast<size_t>(rows) * 2 * sizeof(A)) return kNotApplicable;
  const T* xp = static_cast<const T*>(x);
  A* pairs = static_cast<A*>(scratch);
  const GroupRowMoments<T> op{xp, L};
  hipLaunchKernelGGL((long_rows_sums<T, 1, GroupRowMoments<T>>), dim3(long_rows_grid(rows)),
                     dim3(kLongThreads), 0, stream, rows, static_cast<int>(L), xp, xp, op, pairs);
  hipLaunchKernelGGL((group_stats_from_row_sums<T>), dim3(static_cast<unsigned>(ceil_div(rows, 256))),
                     dim3(256), 0, stream, rows, L, A(eps), xp, pairs, static_cast<A*>(mu),
                     static_cast<A*>(rsig));
  return status_of_launch();
}

template <typename T>
int group_norm_stats_nhwc(const GroupShape& sh, float eps, const void* x, void* mu, void* rsig,
                          void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  const T* xp = static_cast<const T*>(x);
  A* part = static_cast<A*>(scratch);
  A* sums = part + batched_partial_pairs(sh.N, sh.S, sh.C) * 2;
  const BatchedColumns d = launch_batched_columns<T, 1>(
      sh, xp, xp, ColumnStatsAccum<T>{xp, sh.S, sh.C, A(0)}, part, stream);
  hipLaunchKernelGGL((sum_batched_partials<A>),
                     dim3(static_cast<unsigned>(ceil_div(sh.N * sh.C, 256))), dim3(256), 0, stream,
                     d, part, sums);
  hipLaunchKernelGGL((group_stats_from_column_sums<T>),
                     dim3(static_cast<unsigned>(ceil_div(sh.N * sh.G, 256))), dim3(256), 0, stream,
                     d, sh.G, sh.D, A(eps), xp, sums, static_cast<A*>(mu), static_cast<A*>(rsig));
  return status_of_launch();
}

// [N, G, D, 1] and [N, 1, G, D] are the same memory: with S == 1 a group is a
// contiguous row of D elements whatever the layout tag says.
inline int canonical_layout(int layout, int64_t S) {
  return (layout == DRAGON_HIP_NHWC && S == 1) ? DRAGON_HIP_NCHW : layout;
}

// `rows_only`: the caller's kernels address a [N, D] matrix (G = S = 1) by row
// with 64-bit offsets, so only N and D have to fit 32 bits, not their product.
int make_shape(int64_t N, int64_t G, int64_t D, int64_t S, int layout, GroupShape* sh,
               bool rows_only = false) {
  if (N < 0 || G <= 0 || D <= 0 || S < 0) return DRAGON_HIP_EINVAL;
  if (layout != DRAGON_HIP_NCHW && layout != DRAGON_HIP_NHWC) return DRAGON_HIP_EINVAL;
  layout = canonical_layout(layout, S);
  if (rows_only && G == 1 && S == 1) {
    if (!fits_int32(N) || !fits_int32(D)) return DRAGON_HIP_EINVAL;
  } else if (!fits_int32(N * G * D * S)) {
    return DRAGON_HIP_EINVAL;
  }
  sh->N = static_cast<uint32_t>(N), sh->G = static_cast<uint32_t>(G);
  sh->D = static_cast<uint32_t>(D), sh->S = static_cast<uint32_t>(S);
  sh->C = static_cast<uint32_t>(G * D);
  sh->nchw = layout == DRAGON_HIP_NCHW;
  return DRAGON_HIP_OK;
}

// Exchange bytes of the sliced NHWC forward (0: the shape does not take that path).
size_t sample_slices_forward_bytes(int dtype, const GroupShape& sh) {
  SampleSlicePlan p{};
  switch (dtype) {
    case DRAGON_HIP_F16: p = plan_sample_slices<f16_t>(sh.S, sh.C, sh.G, sh.D); break;
    case DRAGON_HIP_BF16: p = plan_sample_slices<bf16_t>(sh.S, sh.C, sh.G, sh.D); break;
    case DRAGON_HIP_F32: p = plan_sample_slices<float>(sh.S, sh.C, sh.G, sh.D); break;
    default: break;
  }
  return p.ok && !sh.nchw ? sample_slices_exchange_bytes(sh.N, sh.G, p.K, 4) : 0;
}

template <typename T>
size_t grad_scratch_t(int64_t N, int64_t G, int64_t D, int64_t S, int layout) {
  return group_norm_grad_scratch<T>(N, G, D, S, layout);
}

} // namespace
} // namespace dragon_hip

extern "C" {

int dragon_hip_group_norm(int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
                          const void* x, const void* mu, const void* rsig, const void* gamma,
                          const void* beta, void* y, void* stream) {
  dragon_hip::GroupShape sh;
  const int st = dragon_hip::make_shape(N, G, D, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!x || !mu || !rsig || !gamma || !beta || !y) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_group_norm, sh, x, mu, rsig, gamma, beta, y, s);
}

size_t dragon_hip_group_norm_grad_scratch_bytes(int dtype, int64_t N, int64_t G, int64_t D,
                                                int64_t S, int layout) {
  dragon_hip::GroupShape sh;
  if (dragon_hip::make_shape(N, G, D, S, layout, &sh, true) != DRAGON_HIP_OK || N * S == 0) return 0;
  layout = dragon_hip::canonical_layout(layout, S);
  switch (dtype) {
    case DRAGON_HIP_F16: return dragon_hip::grad_scratch_t<dragon_hip::f16_t>(N, G, D, S, layout);
    case DRAGON_HIP_BF16: return dragon_hip::grad_scratch_t<dragon_hip::bf16_t>(N, G, D, S, layout);
    case DRAGON_HIP_F32: return dragon_hip::grad_scratch_t<float>(N, G, D, S, layout);
    case DRAGON_HIP_F64: return dragon_hip::grad_scratch_t<double>(N, G, D, S, layout);
    default: return 0;
  }
}

int dragon_hip_group_norm_grad(int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
                               const void* x, const void* mu, const void* rsig,
                               const void* gamma, const void* dy, void* ds, void* db,
                               void* dgamma, void* dbeta, void* dx, void* scratch,
                               size_t scratch_bytes, void* stream) {
  dragon_hip::GroupShape sh;
  // LayerNorm backward (G = S = 1) takes matrices of more than 2^31 elements
  const int st = dragon_hip::make_shape(N, G, D, S, layout, &sh, true);
  if (st != DRAGON_HIP_OK) return st;
  if (!dgamma || !dbeta) return DRAGON_HIP_EINVAL;
  const size_t acc = dtype == DRAGON_HIP_F64 ? 8 : 4;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (N * S == 0) {
    // Nothing to reduce: the reference still zero-fills the parameter gradients.
    const int acc_tag = dtype == DRAGON_HIP_F64 ? DRAGON_HIP_F64 : DRAGON_HIP_F32;
    const int e1 = dragon_hip_set(acc_tag, G * D, 0.f, dgamma, s);
    return e1 != DRAGON_HIP_OK ? e1 : dragon_hip_set(acc_tag, G * D, 0.f, dbeta, s);
  }
  if (!x || !mu || !rsig || !gamma || !dy || !ds || !db || !dx) return DRAGON_HIP_EINVAL;
  // ds == db selects the packed 2*N*G scratch convention of the operator.
  void* db_eff = ds == db ? static_cast<char*>(ds) + acc * N * G : db;
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_group_norm_grad, sh, x, mu, rsig, gamma, dy,
                            ds, db_eff, dgamma, dbeta, dx, scratch, scratch_bytes, s);
}

int dragon_hip_group_norm_grad_timeline(int dtype, int64_t N, int64_t G, int64_t D, int64_t S,
                                        int layout, const void* x, const void* mu, const void* rsig,
                                        const void* gamma, const void* dy, void* ds, void* db,
                                        void* dgamma, void* dbeta, void* dx, void* scratch,
                                        size_t scratch_bytes, void* stamps, size_t workgroups,
                                        void* stream) {
  if (!stamps || workgroups == 0) return DRAGON_HIP_EINVAL;
  dragon_hip::TimelineTarget& target = dragon_hip::timeline_target();
  target.stamps = static_cast<unsigned long long*>(stamps);
  target.workgroups = workgroups;
  const int st = dragon_hip_group_norm_grad(dtype, N, G, D, S, layout, x, mu, rsig, gamma, dy, ds, db,
                                            dgamma, dbeta, dx, scratch, scratch_bytes, stream);
  target.stamps = nullptr;
  target.workgroups = 0;
  return st;
}


namespace {
// Moments view of the group statistics: NCHW [N*G, D*S] over axis 1, NHWC
// [N, S, G, D] over axes {1, 3} (dragon/operators/normalization/group_norm_op.cc:26-34).
struct GroupMomentsView {
  int num_dims, num_axes;
  int64_t dims[4], axes[2];
};
GroupMomentsView group_moments_view(int64_t N, int64_t G, int64_t D, int64_t S, int layout) {
  GroupMomentsView v;
  if (layout == DRAGON_HIP_NCHW) {
    v.num_dims = 2, v.num_axes = 1;
    v.dims[0] = N * G, v.dims[1] = D * S, v.axes[0] = 1;
  } else {
    v.num_dims = 4, v.num_axes = 2;
    v.dims[0] = N, v.dims[1] = S, v.dims[2] = G, v.dims[3] = D;
    v.axes[0] = 1, v.axes[1] = 3;
  }
  return v;
}
} // namespace

size_t dragon_hip_group_norm_forward_scratch_bytes(int dtype, int64_t N, int64_t G, int64_t D,
                                                   int64_t S, int layout) {
  dragon_hip::GroupShape sh;
  if (dragon_hip::make_shape(N, G, D, S, layout, &sh) != DRAGON_HIP_OK || N * S == 0) return 0;
  layout = dragon_hip::canonical_layout(layout, S);
  const GroupMomentsView v = group_moments_view(N, G, D, S, layout);
  size_t bytes = dragon_hip_moments_scratch_bytes(dtype, v.num_dims, v.dims, v.num_axes, v.axes);
  if (layout == DRAGON_HIP_NHWC) {
    const size_t nhwc = (dragon_hip::batched_partial_pairs(N, S, G * D) +
                         static_cast<size_t>(N) * G * D) * 2 * (dtype == DRAGON_HIP_F64 ? 8 : 4);
    if (nhwc > bytes) bytes = nhwc;
    const size_t sliced = dragon_hip::sample_slices_forward_bytes(dtype, sh);
    if (sliced > bytes) bytes = sliced;
  } else {
    const size_t slices = dragon_hip::group_slices_scratch_bytes(dtype, sh);
    if (slices > bytes) bytes = slices;
    // one pair per group row for the one-wavefront-per-row statistics
    const size_t rows = static_cast<size_t>(N) * G * 2 * (dtype == DRAGON_HIP_F64 ? 8 : 4);
    if (rows > bytes) bytes = rows;
  }
  return bytes;
}

int dragon_hip_group_norm_forward(int dtype, int64_t N, int64_t G, int64_t D, int64_t S,
                                  int layout, float eps, const void* x, const void* gamma,
                                  const void* beta, void* mu, void* rsig, void* y,
                                  void* scratch, size_t scratch_bytes, void* stream) {
  dragon_hip::GroupShape sh;
  int st = dragon_hip::make_shape(N, G, D, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  layout = dragon_hip::canonical_layout(layout, S);
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!x || !gamma || !beta || !mu || !rsig || !y) return DRAGON_HIP_EINVAL;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (sh.nchw) {
    // Groups of 32 KB and more that 256 or 512 threads hold whole: two or four workgroups per
    // compute unit, each requesting its next group while it stores, ahead of one 1024-thread
    // workgroup with two register sets (bf16 groups of 128 KB: 49.9 -> 47.5 us).
    switch (dtype) {
      case DRAGON_HIP_F16: st = dragon_hip::try_group_norm_forward_items<dragon_hip::f16_t>(N, G, D, S, eps, x, gamma, beta, mu, rsig, y, hs); break;
      case DRAGON_HIP_BF16: st = dragon_hip::try_group_norm_forward_items<dragon_hip::bf16_t>(N, G, D, S, eps, x, gamma, beta, mu, rsig, y, hs); break;
      case DRAGON_HIP_F32: st = dragon_hip::try_group_norm_forward_items<float>(N, G, D, S, eps, x, gamma, beta, mu, rsig, y, hs); break;
      default: st = dragon_hip::kNotApplicable; break;
    }
    if (st != dragon_hip::kNotApplicable) return st;
  }
  bool fused = false;
  switch (dtype) {
    case DRAGON_HIP_F16:
      fused = dragon_hip::try_group_norm_forward_rows<dragon_hip::f16_t>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
      break;
    case DRAGON_HIP_BF16:
      fused = dragon_hip::try_group_norm_forward_rows<dragon_hip::bf16_t>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
      break;
    case DRAGON_HIP_F32:
      fused = dragon_hip::try_group_norm_forward_rows<float>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
      break;
    case DRAGON_HIP_F64:
      fused = dragon_hip::try_group_norm_forward_rows<double>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
      break;
    default:
      return DRAGON_HIP_EDTYPE;
  }
  if (!fused && !sh.nchw && S > 1) {
    // Channels-last samples go to the slice kernel first, also where one 1024-thread workgroup
    // could hold them: four 256-thread workgroups per compute unit overlap their phases, one
    // workgroup of 1024 does not. A sample of several slices needs scratch for the exchange;
    // without it (and for rows the slice kernel does not take) the one-workgroup kernel stays.
    switch (dtype) {
      case DRAGON_HIP_F16: st = dragon_hip::try_group_norm_forward_nhwc_slices<dragon_hip::f16_t>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      case DRAGON_HIP_BF16: st = dragon_hip::try_group_norm_forward_nhwc_slices<dragon_hip::bf16_t>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      case DRAGON_HIP_F32: st = dragon_hip::try_group_norm_forward_nhwc_slices<float>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      default: st = dragon_hip::kNotApplicable; break;
    }
    if (st != dragon_hip::kNotApplicable) return st;
  }
  if (!fused) {
    switch (dtype) {
      case DRAGON_HIP_F16:
        fused = dragon_hip::try_group_norm_forward_nhwc_samples<dragon_hip::f16_t>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
        break;
      case DRAGON_HIP_BF16:
        fused = dragon_hip::try_group_norm_forward_nhwc_samples<dragon_hip::bf16_t>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
        break;
      case DRAGON_HIP_F32:
        fused = dragon_hip::try_group_norm_forward_nhwc_samples<float>(sh, eps, x, gamma, beta, mu, rsig, y, hs);
        break;
      default:
        break;
    }
  }
  if (fused) return dragon_hip::status_of_launch();
  switch (dtype) {
    case DRAGON_HIP_F16: st = dragon_hip::try_group_norm_forward_slices<dragon_hip::f16_t>(sh, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
    case DRAGON_HIP_BF16: st = dragon_hip::try_group_norm_forward_slices<dragon_hip::bf16_t>(sh, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
    case DRAGON_HIP_F32: st = dragon_hip::try_group_norm_forward_slices<float>(sh, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
    default: st = dragon_hip::try_group_norm_forward_slices<double>(sh, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
  }
  if (st != dragon_hip::kNotApplicable) return st;
  if (!sh.nchw && S > 1) {
    // NHWC: statistics from full-width column reductions of each sample
    if (!scratch || scratch_bytes < dragon_hip_group_norm_forward_scratch_bytes(dtype, N, G, D, S, layout)) {
      return DRAGON_HIP_ESCRATCH;
    }
    // samples beyond one workgroup's registers: slices that exchange their groups' statistics
    switch (dtype) {
      case DRAGON_HIP_F16: st = dragon_hip::try_group_norm_forward_nhwc_slices<dragon_hip::f16_t>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      case DRAGON_HIP_BF16: st = dragon_hip::try_group_norm_forward_nhwc_slices<dragon_hip::bf16_t>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      case DRAGON_HIP_F32: st = dragon_hip::try_group_norm_forward_nhwc_slices<float>(sh.N, sh.S, sh.C, sh.G, sh.D, eps, x, gamma, beta, mu, rsig, y, scratch, scratch_bytes, hs); break;
      default: st = dragon_hip::kNotApplicable; break;
    }
    if (st != dragon_hip::kNotApplicable) return st;
    switch (dtype) {
      case DRAGON_HIP_F16: st = dragon_hip::group_norm_stats_nhwc<dragon_hip::f16_t>(sh, eps, x, mu, rsig, scratch, hs); break;
      case DRAGON_HIP_BF16: st = dragon_hip::group_norm_stats_nhwc<dragon_hip::bf16_t>(sh, eps, x, mu, rsig, scratch, hs); break;
      case DRAGON_HIP_F32: st = dragon_hip::group_norm_stats_nhwc<float>(sh, eps, x, mu, rsig, scratch, hs); break;
      default: st = dragon_hip::group_norm_stats_nhwc<double>(sh, eps, x, mu, rsig, scratch, hs); break;
    }
    if (st != DRAGON_HIP_OK) return st;
    return dragon_hip_group_norm(dtype, N, G, D, S, layout, x, mu, rsig, gamma, beta, y, stream);
  }
  switch (dtype) {
    case DRAGON_HIP_F16: st = dragon_hip::try_group_norm_stats_rows<dragon_hip::f16_t>(sh, eps, x, mu, rsig, scratch, scratch_bytes, hs); break;
    case DRAGON_HIP_BF16: st = dragon_hip::try_group_norm_stats_rows<dragon_hip::bf16_t>(sh, eps, x, mu, rsig, scratch, scratch_bytes, hs); break;
    case DRAGON_HIP_F32: st = dragon_hip::try_group_norm_stats_rows<float>(sh, eps, x, mu, rsig, scratch, scratch_bytes, hs); break;
    default: st = dragon_hip::try_group_norm_stats_rows<double>(sh, eps, x, mu, rsig, scratch, scratch_bytes, hs); break;
  }
  if (st == DRAGON_HIP_OK) {
    return dragon_hip_group_norm(dtype, N, G, D, S, layout, x, mu, rsig, gamma, beta, y, stream);
  }
  if (st != dragon_hip::kNotApplicable) return st;
  const GroupMomentsView v = group_moments_view(N, G, D, S, layout);
  st = dragon_hip_moments(dtype, v.num_dims, v.dims, v.num_axes, v.axes, x, mu, rsig, scratch,
                          scratch_bytes, stream);
  if (st != DRAGON_HIP_OK) return st;
  const int acc_tag = dtype == DRAGON_HIP_F64 ? DRAGON_HIP_F64 : DRAGON_HIP_F32;
  st = dragon_hip_inv_std(acc_tag, N * G, eps, rsig, rsig, stream);
  if (st != DRAGON_HIP_OK) return st;
  return dragon_hip_group_norm(dtype, N, G, D, S, layout, x, mu, rsig, gamma, beta, y, stream);
}

} // extern "C"
