// Single-pass forward and backward of the EMA scan with the tile held in registers.
//
// The scan is HBM-bound and needs one multiply-add per element, so the single-pass kernels
// form no decay matrices: a workgroup owns a tile of 128 rows x BN columns; wave g owns the
// RPL consecutive rows RPL*g .. of it and lane l the CPL adjacent columns CPL*l .., so every
// load or store instruction of a wave moves one contiguous row segment of 64*CPL elements
// and a lane has only RPL short loads in flight (the shape that measured closest to a plain
// device copy on this part).  Each lane runs the recurrence y = a*y + x down its rows:
//
//   1. local pass from a zero state; the value after the last row is what the row group
//      contributes;
//   2. the row groups of the tile are combined per column through LDS, which gives the
//      tile's aggregate; it is published and the state entering the tile is obtained from
//      the earlier tiles of the same columns by the chained scan with look-back (see
//      ema_chain_kernels.h: 64-bit {flag, value} words, ticket order);
//   3. final pass: the recurrence again from the true state entering the row group, stored
//      from registers.  The values are those of the sequential recurrence in float32,
//      whatever the chunking.
//
// The backward does the same from the last row to the first for dx = dy + a[next]*dx[next],
// keeps the forward values y (float32, from the states the forward pass saved) in registers
// and forms dA[m] = a[m] * <dx[m], y[m-1]> on the way.
//
// Two forms of the recurrence (template flag XP):
//   log-decay form   y = a*y + x,        a = exp(min(A, 0));   gradients dx = r, dA = a*<r, y_prev>
//   probability form y = (1-p)*y + p*x,  evaluated as y + p*(x - y);  dx = p*r, dp = <r, x - y_prev>
// with r the reverse scan of dy.  In the probability form a set sign bit on p (-p, or -0.0 for
// p = 0) marks the first position of a packed sequence: the state is dropped there, y = p*x,
// and the gradient returned for such a coefficient is that of the encoded value, -<r, x>.  (In
// the log-decay form the same is a decay of exp(-inf) = 0 and needs no flag.)
// The state before the first row may be given (init) and the
// gradient reaching the state after the last row (dfinal); the backward then also returns the
// gradient of the initial state, a[0]*r[0].
#pragma once
#include "ema_chain_kernels.h"

namespace ema {

#ifdef EMA_TIMING
// Development builds only: one thread per role keeps up to 8 timestamps per tile in registers and
// writes them out when the tile is finished, so that taking a stamp waits for nothing.  A tile has
// 16 slots in the buffer: 0..7 for thread 0 of the workgroup, 8..15 for the thread `EMA_TS_ROW`
// (the first thread of a wave that only owns rows, where a kernel has such waves).
#define EMA_TSTAMP_DECL long long ema_ts[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define EMA_TSTAMP_T(tid, slot)                            \
  do {                                                     \
    if (threadIdx.x == (tid)) ema_ts[slot] = wall_clock64(); \
  } while (0)
#define EMA_TSTAMP(slot) EMA_TSTAMP_T(0, slot)
#define EMA_TSTAMP_VALUE(slot, v)             \
  do {                                        \
    if (threadIdx.x == 0) ema_ts[slot] = (v); \
  } while (0)
#define EMA_TSTAMP_FLUSH_T(tid, base)                                                  \
  do {                                                                                 \
    if (threadIdx.x == (tid) && g_ema_timing)                                          \
      for (int q = 0; q < 8; ++q) g_ema_timing[(int64_t)cur * 16 + (base) + q] = ema_ts[q]; \
  } while (0)
#define EMA_TSTAMP_FLUSH EMA_TSTAMP_FLUSH_T(0, 0)
#else
#define EMA_TSTAMP_DECL \
  do {                  \
  } while (0)
#define EMA_TSTAMP_T(tid, slot) \
  do {                          \
  } while (0)
#define EMA_TSTAMP(slot) \
  do {                   \
  } while (0)
#define EMA_TSTAMP_VALUE(slot, v) \
  do {                            \
  } while (0)
#define EMA_TSTAMP_FLUSH_T(tid, base) \
  do {                                \
  } while (0)
#define EMA_TSTAMP_FLUSH \
  do {                   \
  } while (0)
#endif

// Which accesses of the single-pass kernels are non-temporal (the sequences are touched once per
// kernel): bit 0 forward loads, bit 1 forward stores, bit 2 backward loads, bit 3 backward
// stores.  Measured at b16 nh2 d1024 L4096: forward 126 -> 119 us with both, backward 184 -> 176 us
// with the loads; non-temporal stores cost the backward 1 %.
#ifndef EMA_STREAM_FLAGS
#define EMA_STREAM_FLAGS 0x7
#endif
constexpr bool kStreamFwdLoad = (EMA_STREAM_FLAGS & 1) != 0, kStreamFwdStore = (EMA_STREAM_FLAGS & 2) != 0,
               kStreamBwdLoad = (EMA_STREAM_FLAGS & 4) != 0, kStreamBwdStore = (EMA_STREAM_FLAGS & 8) != 0;

// Output rows are written through to device memory (1) instead of being left to the L2s' write-back
// (0).  Measured at b16 nh2 d1024 L4096: forward 112 -> 105 us, step 279 -> 271 us.
#ifndef EMA_STORE_WT
#define EMA_STORE_WT 1
#endif
template <typename T, int CPL, int RPL>
struct TileCfg {
  static constexpr int NG = kTileRows / RPL;            // row groups = waves of the workgroup
  static constexpr int NT = 64 * NG;                    // threads
  static constexpr int BN = 64 * CPL;                   // columns of a tile
  static constexpr int NW = CPL * (int)sizeof(T) / 4;   // 32-bit words of one lane's row
  static_assert(NW == 1 || NW == 2 || NW == 4, "a lane's row is 4, 8 or 16 bytes");
  static_assert(NG * RPL == kTileRows && NG <= 16 && BN <= NT, "tile shape");
};

template <int NW>
struct RowWords {
  unsigned w[NW];
};

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
// STREAM: the data is touched once by this kernel (non-temporal access)
template <int NW, bool STREAM = false>
__device__ __forceinline__ RowWords<NW> row_load(const void* p) {
  RowWords<NW> r;
  if constexpr (NW == 4) {
    const uintx4 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(p))
                            : *reinterpret_cast<const uintx4*>(p);
    r.w[0] = v[0], r.w[1] = v[1], r.w[2] = v[2], r.w[3] = v[3];
  } else if constexpr (NW == 2) {
    const uintx2 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const uintx2*>(p))
                            : *reinterpret_cast<const uintx2*>(p);
    r.w[0] = v[0], r.w[1] = v[1];
  } else {
    r.w[0] = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(p))
                    : *reinterpret_cast<const unsigned*>(p);
  }
  return r;
}
template <int NW, bool STREAM = false>
__device__ __forceinline__ void row_store(void* p, const RowWords<NW>& r) {
  if constexpr (NW == 4) {
    const uintx4 v = {r.w[0], r.w[1], r.w[2], r.w[3]};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<uintx4*>(p));
    else *reinterpret_cast<uintx4*>(p) = v;
  } else if constexpr (NW == 2) {
#if EMA_STORE_WT
    // written through to device memory (a relaxed store at agent scope): nothing of the output
    // stays behind as dirty lines in the L2s for the end of the kernel to write back
    const unsigned long long v = ((unsigned long long)r.w[1] << 32) | r.w[0];
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
    const uintx2 v = {r.w[0], r.w[1]};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<uintx2*>(p));
    else *reinterpret_cast<uintx2*>(p) = v;
#endif
  } else {
    if (STREAM) __builtin_nontemporal_store(r.w[0], reinterpret_cast<unsigned*>(p));
    else *reinterpret_cast<unsigned*>(p) = r.w[0];
  }
}
template <int NW>
__device__ __forceinline__ RowWords<NW> row_zero() {
  RowWords<NW> r;
#pragma unroll
  for (int i = 0; i < NW; ++i) r.w[i] = 0u;
  return r;
}

// element e of a row as float
template <typename T, int NW>
__device__ __forceinline__ float row_get(const RowWords<NW>& r, int e) {
  if constexpr (sizeof(T) == 4) return __uint_as_float(r.w[e]);
  else return __uint_as_float((e & 1) ? (r.w[e >> 1] & 0xffff0000u) : (r.w[e >> 1] << 16));
}

typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
// CPL floats -> a row (round to nearest even for bf16)
template <typename T, int CPL, int NW>
__device__ __forceinline__ RowWords<NW> row_pack(const float* v) {
  RowWords<NW> r;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < NW; ++e) r.w[e] = __float_as_uint(v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < NW; ++e) {
      bf16x2 p;
      p[0] = (bf16_t)v[2 * e];
      p[1] = (bf16_t)v[2 * e + 1];
      r.w[e] = __builtin_bit_cast(unsigned, p);
    }
  }
  return r;
}

// Makes the registers of a tile opaque to the optimiser, so that values derived from them in
// one pass (the float32 conversions) are formed again in the next pass instead of being kept.
template <int NW, int RPL>
__device__ __forceinline__ void rows_opaque(RowWords<NW>* rows) {
#pragma unroll
  for (int i = 0; i < RPL; ++i)
#pragma unroll
    for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(rows[i].w[k]));
}

// Where a workgroup finds its part of a tile of a sequence tensor.
struct TileAt {
  int nrows;  // valid rows of this wave (may be <= 0)
  bool cok;   // this lane's columns lie inside the tensor
  bool full;  // all rows and all lanes of the wave are inside: no per-row predicates needed
};
template <int RPL>
__device__ __forceinline__ TileAt tile_at(int limit, int grp, bool cok) {
  TileAt a;
  a.nrows = limit - RPL * grp;
  a.cok = cok;
  a.full = a.nrows >= RPL && __all(cok);
  return a;
}
// Row i of this lane: g points at (first row of the wave, this lane's first column).  Rows at or
// past nrows and columns past the end read as 0.
template <int NW, bool STREAM, typename T>
__device__ __forceinline__ RowWords<NW> tile_load_row(const T* __restrict__ g, int64_t sl, int i, const TileAt& at) {
  if (at.full) return row_load<NW, STREAM>(g + (int64_t)i * sl);
  return (i < at.nrows && at.cok) ? row_load<NW, STREAM>(g + (int64_t)i * sl) : row_zero<NW>();
}

// A value that is the same in every lane, moved to a scalar register.
__device__ __forceinline__ float wave_uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

// Raw coefficients of the wave's RPL rows (uniform addresses), requested ahead of their use;
// rows at or past nrows get the neutral value (log-decay 0, probability 0).
template <int RPL>
__device__ __forceinline__ void tile_coef_load(float* raw, const float* __restrict__ A, int64_t a_sl, int nrows) {
#pragma unroll
  for (int i = 0; i < RPL; ++i) raw[i] = i < nrows ? A[(int64_t)i * a_sl] : 0.f;
}
// The same from the inclusive cumsum of the log-decay over the 128-row chunk that the tile is
// (cs points at the wave's first row, dense along the rows): raw[i] = cs[i] - cs[i - 1], and cs[0]
// itself for the chunk's first row.
template <int RPL>
__device__ __forceinline__ void tile_coef_load_cumsum(float* raw, const float* __restrict__ cs, int nrows,
                                                      bool chunk_start) {
  float before = chunk_start ? 0.f : cs[-1];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const float here = i < nrows ? cs[i] : before;
    raw[i] = here - before;
    before = here;
  }
}
// Log-decay form: a[i] = exp(min(A[row], 0)).  Probability form: a[i] = p[row].  Scalar registers.
template <int RPL, bool XP>
__device__ __forceinline__ void tile_decays(float* a, const float* raw) {
#pragma unroll
  for (int i = 0; i < RPL; ++i) a[i] = wave_uniform(XP ? raw[i] : __expf(fminf(raw[i], 0.f)));
}

// Probability form: the sign bit of a coefficient marks the first position of a packed sequence.
__device__ __forceinline__ bool coef_resets(float coef) { return (__float_as_uint(coef) >> 31) != 0u; }

// One step of the forward recurrence, and the factor by which the step scales the state.
template <bool XP>
__device__ __forceinline__ float tile_step(float coef, float s, float x) {
  if (XP) {
    const float s0 = coef_resets(coef) ? 0.f : s;
    return fmaf(fabsf(coef), x - s0, s0);
  }
  return fmaf(coef, s, x);
}
template <bool XP>
__device__ __forceinline__ float tile_keep(float coef) {
  if (XP) return coef_resets(coef) ? 0.f : 1.f - coef;
  return coef;
}

// ------------------------------------------------------------------------------------
// Forward.  Writes y, prev[n,c,:] (state entering each 128-row chunk), optionally a copy at
// a coarser chunking and the final state.  init (may be null): the state before the first row,
// (N, T).  hdr / decw / status: the chained-scan workspace (zero-filled once, see
// ema_chain_kernels.h); decw has N*C words, status N*ntiles*C*BN.  One ticket = one tile; the
// next ticket is fetched while the tile is processed.
//
// Per tile and column the row groups are combined in one chain of NG steps by the workgroup's
// first BN threads (one per column), straight after the local pass: the chain leaves in LDS, for
// every row group, the state entering it if nothing entered the tile, and yields the tile's
// aggregate, which is published at once.  What the look-back then returns enters every group
// scaled by the decay of the groups before it, so the final pass starts from two LDS reads.
// ------------------------------------------------------------------------------------
template <typename T, int CPL, int RPL, int MINW, bool XP>
__global__ __launch_bounds__(64 * (kTileRows / RPL), MINW) void fwd_tile_kernel(
    const T* __restrict__ x, SeqStrides sx, const float* __restrict__ A, SeqStrides sa,
    T* __restrict__ y, SeqStrides sy, float* __restrict__ prev, float* __restrict__ prev_coarse, int ratio,
    float* __restrict__ final_state, const float* __restrict__ init, ChainHeader* __restrict__ hdr,
    u64* __restrict__ decw, u64* __restrict__ status, int nh, int L, int Tdim, int C, int ntiles, int cols,
    int total, const TileOrder ord) {
  using W = TileCfg<T, CPL, RPL>;
  constexpr int BN = W::BN, NW = W::NW, NG = W::NG;
  __shared__ __attribute__((aligned(16))) float sS[2][NG][BN];  // group states, double-buffered by tile
  __shared__ __attribute__((aligned(16))) float sP[2][BN];      // state entering the tile
  __shared__ float sD[2][NG];                                   // total decay of each row group
  __shared__ float sW[2][NG];                                   // decay of the groups before each group
  __shared__ int s_ticket[3];
  const int lane = threadIdx.x & 63;
  const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const unsigned off = (unsigned)lane * CPL;
  const bool looks = grp * 64 < BN;  // this wave's threads own a column each in step 2
  const ChainCtl ctl = chain_enter(hdr);

  if (threadIdx.x == 0) {
    s_ticket[0] = (int)atomicAdd(&hdr->ticket, 1u);
    s_ticket[1] = (int)atomicAdd(&hdr->ticket, 1u);
  }
  __syncthreads();
  int cur = s_ticket[0], nxt = s_ticket[1], buf = 0, slot = 2;

  // Two register sets hold the tile being processed and the one after it: the rows of the next
  // tile are requested right after the first barrier, so they travel while this tile waits for
  // its look-back, makes its final pass and stores.  The waves whose threads look back request
  // theirs after the look-back: loads return in the order of their requests, and a poll queued
  // behind eight row loads would wait for all of them.
  RowWords<NW> rowsA[RPL], rowsB[RPL];
  float arawA[RPL], arawB[RPL];
  auto request = [&](RowWords<NW>* rows, float* araw, const ChainTile& tt, const TileAt& aa) {
    const T* g = x + (int64_t)tt.b * sx.sb + (int64_t)tt.h * sx.sh +
                 ((int64_t)tt.c * kTileRows + RPL * grp) * sx.sl + tt.col0 + off;
#pragma unroll
    for (int i = 0; i < RPL; ++i) rows[i] = tile_load_row<NW, kStreamFwdLoad>(g, sx.sl, i, aa);
    tile_coef_load<RPL>(araw, A + (int64_t)tt.b * sa.sb + (int64_t)tt.h * sa.sh +
                                  ((int64_t)tt.c * kTileRows + RPL * grp) * sa.sl, sa.sl, aa.nrows);
  };
  ChainTile t = chain_decode<false, BN>(cur < total ? cur : 0, ord, L);
  TileAt at = tile_at<RPL>(t.limit, grp, t.col0 + lane * CPL < Tdim);
  if (cur < total) request(rowsA, arawA, t, at);

  // one tile: `rows` / `araw` hold it, `rows_n` / `araw_n` receive the next one
  auto tile = [&](RowWords<NW>* rows, float* araw, RowWords<NW>* rows_n, float* araw_n) {
    int future = 0;
    if (threadIdx.x == 0) future = (int)atomicAdd(&hdr->ticket, 1u);
    const bool more = nxt < total;
    const ChainTile tn = chain_decode<false, BN>(more ? nxt : 0, ord, L);
    const TileAt atn = tile_at<RPL>(tn.limit, grp, tn.col0 + lane * CPL < Tdim);
    EMA_TSTAMP_DECL;
    EMA_TSTAMP(0);
    EMA_TSTAMP_VALUE(7, (long long)blockIdx.x);
    float a[RPL];
    tile_decays<RPL, XP>(a, araw);
    EMA_TSTAMP(5);
    // 1. local pass
    float s[CPL];
    float D = 1.f;
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      D *= tile_keep<XP>(a[i]);
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = tile_step<XP>(a[i], s[e], row_get<T, NW>(rows[i], e));
    }
#pragma unroll
    for (int e = 0; e < CPL; ++e) sS[buf][grp][lane * CPL + e] = s[e];
    if (lane == 0) sD[buf][grp] = D;
    rows_opaque<NW, RPL>(rows);
    __syncthreads();
    EMA_TSTAMP(1);
    if (more && !looks) request(rows_n, araw_n, tn, atn);

    // 2. one thread per column: chain over the row groups, publish, look back
    if (threadIdx.x < BN) {
      const int k = threadIdx.x;
      u64* words = status + ((int64_t)t.col_id * C) * BN + k;
      u64* dws = decw + (int64_t)t.n * C;
      // all reads first (the group decays are the same for every column: scalar registers),
      // then the chain: otherwise every step waits for its own LDS read
      float sg[NG], dg[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) sg[g] = sS[buf][g][k];
#pragma unroll
      for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[buf][g]);
      float loc = 0.f, dec = 1.f;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        sS[buf][g][k] = loc;
        if (k == 0) sW[buf][g] = dec;
        loc = fmaf(dg[g], loc, sg[g]);
        dec *= dg[g];
      }
      float p_in;
      if (t.c > 0) {
        if (k == 0) chain_publish(dws + t.c, ctl.epoch, kStateAggregate, dec);
        chain_publish(words + (int64_t)t.c * BN, ctl.epoch, kStateAggregate, loc);
        ChainLook<false, BN> look;
        EMA_TSTAMP(4);
        look.begin(words, t.c);
        p_in = look.finish(words, dws, C, ctl);
        EMA_TSTAMP(6);
      } else {
        p_in = (init && t.c == 0 && t.col0 + k < Tdim) ? init[(int64_t)t.n * Tdim + t.col0 + k] : 0.f;
      }
      const float p_out = fmaf(dec, p_in, loc);
      chain_publish(words + (int64_t)t.c * BN, ctl.epoch, kStatePrefix, p_out);
      sP[buf][k] = p_in;
      if (t.col0 + k < Tdim) {
        prev[(int64_t)t.chunk_id * Tdim + t.col0 + k] = p_in;
        if (prev_coarse && t.c % ratio == 0)
          prev_coarse[((int64_t)t.n * ((C + ratio - 1) / ratio) + t.c / ratio) * Tdim + t.col0 + k] = p_in;
        if (final_state && t.c == C - 1) final_state[(int64_t)t.n * Tdim + t.col0 + k] = p_out;
      }
    }
    if (more && looks) request(rows_n, araw_n, tn, atn);
    if (threadIdx.x == 0) s_ticket[slot] = future;
    __syncthreads();
    EMA_TSTAMP(2);

    // 3. final pass from the true state
    {
      const float wg = sW[buf][grp];
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = fmaf(wg, sP[buf][lane * CPL + e], sS[buf][grp][lane * CPL + e]);
      T* g = y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh +
             ((int64_t)t.c * kTileRows + RPL * grp) * sy.sl + t.col0 + off;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = tile_step<XP>(a[i], s[e], row_get<T, NW>(rows[i], e));
        if (i < at.nrows && at.cok) row_store<NW, kStreamFwdStore>(g + (int64_t)i * sy.sl, row_pack<T, CPL, NW>(s));
      }
    }
    EMA_TSTAMP(3);
    EMA_TSTAMP_FLUSH;
    cur = nxt;
    nxt = s_ticket[slot];
    t = tn;
    at = atn;
    slot = slot == 2 ? 0 : slot + 1;
    buf ^= 1;
  };
  while (cur < total) {
    tile(rowsA, arawA, rowsB, arawB);
    if (cur >= total) break;
    tile(rowsB, arawB, rowsA, arawA);
  }
  if (threadIdx.x == 0) chain_leave(hdr, ctl);
}

// ------------------------------------------------------------------------------------
// Backward.  prev[n,c,:] (states entering each 128-row chunk, from the forward) is an input;
// the reverse state entering each tile from the rows after it, H = a[next row] * dx[next row],
// comes from the chained scan over dy, last chunk first.  Writes dx, optionally y, and the
// column partials part[(chunk*ntiles + ctile)*128 + m] = a[m] * <dx[m], y[m-1]> over the
// tile's columns (probability form: <r[m], x[m] - y[m-1]>).  dfinal (may be null): the gradient
// reaching the state after the last row, (N, T); dinit (may be null) receives the gradient of
// the state before the first.
//
// After the local passes the first BN threads chain the reverse group states (and publish the
// aggregate), the next BN threads chain the forward group states from the saved chunk-entry
// state; the forward values y are then recomputed while the reverse look-back is under way.
// As in the forward, the rows of the next tile are requested behind the stores of this one.
// ------------------------------------------------------------------------------------
//
// GIVEN: the reverse state entering every tile is an input as well (given[n,c,:], the gradient of the
// state that leaves chunk c, as the reverse state passing of the per-stage path computes it), and A
// is the per-chunk inclusive cumsum of the log-decay, dense (N, C, 128), described by sa.  Nothing
// is chained then: no workspace words, no tickets (workgroup w takes the tiles w, w + grid, ...), and
// hdr / decw / status are not touched.
template <typename T, int CPL, int RPL, int MINW, bool WRITE_Y, bool XP, bool GIVEN = false>
__global__ __launch_bounds__(64 * (kTileRows / RPL), MINW) void bwd_tile_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ A, SeqStrides sa, const float* __restrict__ prev, T* __restrict__ dx,
    SeqStrides sdx, T* __restrict__ y, SeqStrides sy, float* __restrict__ part,
    const float* __restrict__ dfinal, float* __restrict__ dinit, ChainHeader* __restrict__ hdr,
    u64* __restrict__ decw, u64* __restrict__ status, int nh, int L, int Tdim, int C, int ntiles, int cols,
    int total, const TileOrder ord, const float* __restrict__ given = nullptr) {
  static_assert(!(GIVEN && XP), "the given-state form reads a cumsum of log-decays");
  using W = TileCfg<T, CPL, RPL>;
  constexpr int BN = W::BN, NW = W::NW, NG = W::NG, NT = W::NT;
  static_assert(2 * BN <= NT, "one thread per column and direction");
  __shared__ __attribute__((aligned(16))) float sS[2][NG][BN];  // forward group states
  __shared__ __attribute__((aligned(16))) float sR[2][NG][BN];  // reverse group states
  __shared__ __attribute__((aligned(16))) float sH[2][BN];      // reverse state entering the tile
  __shared__ float sD[2][NG];
  __shared__ float sW[2][NG];  // decay of the groups after each group
  __shared__ int s_ticket[2];
  const int lane = threadIdx.x & 63;
  const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const unsigned off = (unsigned)lane * CPL;
  const int kf = (int)threadIdx.x - BN;  // column of the threads that chain the forward group states
  ChainCtl ctl;
  if constexpr (!GIVEN) {
    ctl = chain_enter(hdr);
    if (threadIdx.x == 0) s_ticket[0] = (int)atomicAdd(&hdr->ticket, 1u);
    __syncthreads();
  }
  int cur = GIVEN ? (int)blockIdx.x : s_ticket[0], buf = 0, slot = 1;
  // the coefficients of this wave's rows of tile tt
  auto coef_load = [&](float* raw, const ChainTile& tt, int64_t row, int nrows) {
    const float* ap = A + (int64_t)tt.b * sa.sb + (int64_t)tt.h * sa.sh + row * sa.sl;
    if constexpr (GIVEN) tile_coef_load_cumsum<RPL>(raw, ap, nrows, grp == 0);
    else tile_coef_load<RPL>(raw, ap, sa.sl, nrows);
  };
  RowWords<NW> dr[RPL], xr[RPL];
  float araw[RPL];
  float p_in = 0.f;
  ChainTile t = chain_decode<true, BN>(cur < total ? cur : 0, ord, L);
  TileAt at = tile_at<RPL>(t.limit, grp, t.col0 + lane * CPL < Tdim);
  if (cur < total) {
    const int64_t row0 = (int64_t)t.c * kTileRows + RPL * grp;
    const T* gd = dy + (int64_t)t.b * sd.sb + (int64_t)t.h * sd.sh + row0 * sd.sl + t.col0 + off;
    const T* gx = x + (int64_t)t.b * sx.sb + (int64_t)t.h * sx.sh + row0 * sx.sl + t.col0 + off;
#pragma unroll
    for (int i = 0; i < RPL; ++i) dr[i] = tile_load_row<NW, kStreamBwdLoad>(gd, sd.sl, i, at);
#pragma unroll
    for (int i = 0; i < RPL; ++i) xr[i] = tile_load_row<NW, kStreamBwdLoad>(gx, sx.sl, i, at);
    coef_load(araw, t, row0, at.nrows);
    if (kf >= 0 && kf < BN && t.col0 + kf < Tdim) p_in = prev[(int64_t)t.chunk_id * Tdim + t.col0 + kf];
  }
  while (cur < total) {
    int future = GIVEN ? cur + (int)gridDim.x : 0;
    if constexpr (!GIVEN) {
      if (threadIdx.x == 0) future = (int)atomicAdd(&hdr->ticket, 1u);
    }
    EMA_TSTAMP_DECL;
    EMA_TSTAMP(0);
    EMA_TSTAMP_VALUE(7, (long long)blockIdx.x);
    const int64_t row0 = (int64_t)t.c * kTileRows + RPL * grp;
    // a: factor of the state per row; pc: the row's coefficient as tile_step takes it
    float a[RPL], pc[RPL];
    tile_decays<RPL, XP>(pc, araw);
    EMA_TSTAMP(5);
#pragma unroll
    for (int i = 0; i < RPL; ++i) a[i] = tile_keep<XP>(pc[i]);

    // 1a. local reverse pass over dy, r = a[i] * dx_local[i]; at the end the state that the
    // group hands to the rows before it
    float r[CPL], s[CPL];
    float D = 1.f;
#pragma unroll
    for (int e = 0; e < CPL; ++e) r[e] = 0.f, s[e] = 0.f;
#pragma unroll
    for (int i = RPL - 1; i >= 0; --i) {
      D *= a[i];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = a[i] * (row_get<T, NW>(dr[i], e) + r[e]);
    }
    // 1b. local forward pass over x
#pragma unroll
    for (int i = 0; i < RPL; ++i)
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = tile_step<XP>(pc[i], s[e], row_get<T, NW>(xr[i], e));
#pragma unroll
    for (int e = 0; e < CPL; ++e) {
      sR[buf][grp][lane * CPL + e] = r[e];
      sS[buf][grp][lane * CPL + e] = s[e];
    }
    if (lane == 0) sD[buf][grp] = D;
    rows_opaque<NW, RPL>(dr);
    rows_opaque<NW, RPL>(xr);
    __syncthreads();
    EMA_TSTAMP(1);

    // 2a. chains over the row groups, one thread per column and direction
    u64* words = status + ((int64_t)t.col_id * C) * BN + (threadIdx.x < BN ? (int)threadIdx.x : 0);
    u64* dws = decw + (int64_t)t.n * C;
    const bool last = t.c == C - 1;
    float loc = 0.f, dec = 1.f;
    ChainLook<true, BN> look;
    if (threadIdx.x < BN) {
      const int k = threadIdx.x;
      float rg[NG], dg[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) rg[g] = sR[buf][g][k];
#pragma unroll
      for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[buf][g]);
#pragma unroll
      for (int g = NG - 1; g >= 0; --g) {
        sR[buf][g][k] = loc;
        if (k == 0) sW[buf][g] = dec;
        loc = fmaf(dg[g], loc, rg[g]);
        dec *= dg[g];
      }
      if constexpr (!GIVEN) {
        if (!last) {
          if (k == 0) chain_publish(dws + t.c, ctl.epoch, kStateAggregate, dec);
          chain_publish(words + (int64_t)t.c * BN, ctl.epoch, kStateAggregate, loc);
          look.begin(words, t.c);
        }
      }
    } else if (kf < BN) {
      float sg[NG], dg[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) sg[g] = sS[buf][g][kf];
#pragma unroll
      for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[buf][g]);
      float E = p_in;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        sS[buf][g][kf] = E;
        E = fmaf(dg[g], E, sg[g]);
      }
    }
    __syncthreads();
    EMA_TSTAMP(2);

    // 1c. forward values y from the true state (kept in float32 for the dots)
    float E[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) E[e] = sS[buf][grp][lane * CPL + e];
    float yv[RPL][CPL];
    {
      T* g = WRITE_Y ? y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + row0 * sy.sl + t.col0 + off : nullptr;
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = E[e];
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
#pragma unroll
        for (int e = 0; e < CPL; ++e) {
          s[e] = tile_step<XP>(pc[i], s[e], row_get<T, NW>(xr[i], e));
          yv[i][e] = s[e];
        }
        if (WRITE_Y && i < at.nrows && at.cok) row_store<NW>(g + (int64_t)i * sy.sl, row_pack<T, CPL, NW>(s));
      }
    }
    // Given-state form: the x rows of the next tile are requested here, where this tile's have been
    // used for the last time, and not behind the stores of the final pass (0.159 -> 0.152 ms at b16
    // nh2 d1024 L4096).  The chained form must not: rows requested while the look-back is under way
    // slow its polls down, and everybody waits for those (158 -> 163 us).
    if constexpr (GIVEN) {
      if (future < total) {
        const ChainTile tx = chain_decode<true, BN>(future, ord, L);
        const TileAt atx = tile_at<RPL>(tx.limit, grp, tx.col0 + lane * CPL < Tdim);
        const T* gx = x + (int64_t)tx.b * sx.sb + (int64_t)tx.h * sx.sh +
                      ((int64_t)tx.c * kTileRows + RPL * grp) * sx.sl + tx.col0 + off;
#pragma unroll
        for (int i = 0; i < RPL; ++i) xr[i] = tile_load_row<NW, kStreamBwdLoad>(gx, sx.sl, i, atx);
      }
    }

    // 2b. the reverse state entering the tile (the waves that own no column go straight on)
    if (threadIdx.x < BN) {
      const int k = threadIdx.x;
      float h_in;
      if constexpr (GIVEN) {
        h_in = t.col0 + k < Tdim ? given[(int64_t)t.chunk_id * Tdim + t.col0 + k] : 0.f;
      } else {
        if (!last) h_in = look.finish(words, dws, C, ctl);
        else h_in = (dfinal && last && t.col0 + k < Tdim) ? dfinal[(int64_t)t.n * Tdim + t.col0 + k] : 0.f;
        EMA_TSTAMP(6);
        const float h_out = fmaf(dec, h_in, loc);
        chain_publish(words + (int64_t)t.c * BN, ctl.epoch, kStatePrefix, h_out);
        if (dinit && t.c == 0 && t.col0 + k < Tdim) dinit[(int64_t)t.n * Tdim + t.col0 + k] = h_out;
      }
      sH[buf][k] = h_in;
    }
    if constexpr (!GIVEN) {
      if (threadIdx.x == 0) s_ticket[slot] = future;
    }
    __syncthreads();
    EMA_TSTAMP(3);

    // 3. final reverse pass: dx, and the dots with the row before; behind each stored row the
    // same rows of the next tile are requested
    const int next = GIVEN ? future : s_ticket[slot];
    const bool more = next < total;
    const ChainTile tn = chain_decode<true, BN>(more ? next : 0, ord, L);
    const TileAt atn = tile_at<RPL>(tn.limit, grp, tn.col0 + lane * CPL < Tdim);
    {
      T* g = dx + (int64_t)t.b * sdx.sb + (int64_t)t.h * sdx.sh + row0 * sdx.sl + t.col0 + off;
      const int64_t rown = (int64_t)tn.c * kTileRows + RPL * grp;
      const T* gd = dy + (int64_t)tn.b * sd.sb + (int64_t)tn.h * sd.sh + rown * sd.sl + tn.col0 + off;
      const T* gx = x + (int64_t)tn.b * sx.sb + (int64_t)tn.h * sx.sh + rown * sx.sl + tn.col0 + off;
      float dA = 0.f;  // lane i reports row i of the wave
      const float wg = sW[buf][grp];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = fmaf(wg, sH[buf][lane * CPL + e], sR[buf][grp][lane * CPL + e]);
#pragma unroll
      for (int i = RPL - 1; i >= 0; --i) {
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < CPL; ++e) {
          // r holds a[i+1] * dx[i+1] on entry (the carried state for the last row)
          const float d = row_get<T, NW>(dr[i], e) + r[e];
          float yp = i > 0 ? yv[i - 1][e] : E[e];
          if (XP && coef_resets(pc[i])) yp = 0.f;
          dot = fmaf(d, XP ? row_get<T, NW>(xr[i], e) - yp : yp, dot);
          r[e] = d;
        }
        if (XP) {
          float o[CPL];
#pragma unroll
          for (int e = 0; e < CPL; ++e) o[e] = fabsf(pc[i]) * r[e];
          if (i < at.nrows && at.cok) row_store<NW, kStreamBwdStore>(g + (int64_t)i * sdx.sl, row_pack<T, CPL, NW>(o));
        } else {
          if (i < at.nrows && at.cok) row_store<NW, kStreamBwdStore>(g + (int64_t)i * sdx.sl, row_pack<T, CPL, NW>(r));
        }
        if (more) {
          dr[i] = tile_load_row<NW, kStreamBwdLoad>(gd, sd.sl, i, atn);
          if (!GIVEN) xr[i] = tile_load_row<NW, kStreamBwdLoad>(gx, sx.sl, i, atn);
        }
#pragma unroll
        for (int e = 0; e < CPL; ++e) r[e] *= a[i];
        dot = wave_sum(dot);
        if (!XP) dot *= a[i];
        else if (coef_resets(pc[i])) dot = -dot;  // derivative with respect to the encoded value -p
        if (lane == i) dA = dot;
      }
      if (lane < RPL)
        part[((int64_t)t.chunk_id * ntiles + t.ctile) * kTileRows + RPL * grp + lane] = lane < at.nrows ? dA : 0.f;
      if (more) {
        coef_load(araw, tn, rown, atn.nrows);
        p_in = (kf >= 0 && kf < BN && tn.col0 + kf < Tdim) ? prev[(int64_t)tn.chunk_id * Tdim + tn.col0 + kf] : 0.f;
      }
    }
    EMA_TSTAMP(4);
    EMA_TSTAMP_FLUSH;
    cur = next;
    t = tn;
    at = atn;
    slot ^= 1;
    buf ^= 1;
  }
  if constexpr (!GIVEN) {
    if (threadIdx.x == 0) chain_leave(hdr, ctl);
  }
}

// out[b, p, h] = sum over the column tiles of part[n, p / 128, tile, p % 128]: the gradient of
// the per-position coefficient in the layout of the coefficient itself.  One thread per (n, p).
__global__ __launch_bounds__(256) void dcoef_reduce_kernel(const float* __restrict__ part,
                                                           float* __restrict__ out, SeqStrides so, int nh,
                                                           int L, int Ci, int ntiles, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t n = i / L;
  const int64_t p = i - n * L;
  const int64_t ci = p / kTileRows;
  const int q = (int)(p - ci * kTileRows);
  const float* pp = part + ((n * Ci + ci) * ntiles) * (int64_t)kTileRows + q;
  float s = 0.f;
  for (int t = 0; t < ntiles; ++t) s += pp[(int64_t)t * kTileRows];
  const int64_t b = n / nh;
  const int64_t h = n - b * nh;
  out[b * so.sb + p * so.sl + h * so.sh] = s;
}

}  // namespace ema
