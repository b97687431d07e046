// Single-pass forward and backward of the EMA scan with the tile of a wave held in registers.
//
// The scan is HBM-bound and needs one multiply-add per element, so the single-pass kernels do
// not form decay matrices at all: a wave owns a tile of 128 rows x BN columns, each lane owns
// 32 consecutive rows of CPL adjacent columns (lane l: rows 32*(l/16).., columns CPL*(l%16)..),
// loads them straight into registers and runs the recurrence y = a*y + x down its rows.
//
//   1. local pass: every lane scans its 32 rows from a zero state; the result at the last row
//      is the state its row group contributes;
//   2. the four row groups of the tile are combined through a few hundred bytes of LDS, which
//      gives the tile's aggregate; the aggregate is published and the state entering the tile
//      is obtained from the earlier tiles of the same columns by the chained scan with
//      look-back (see ema_chain_kernels.h: 64-bit {flag, value} words, ticket order);
//   3. final pass: every lane runs the recurrence again from the true state entering its row
//      group and stores the results from registers.  The values are those of the sequential
//      recurrence in float32, whatever the chunking.
//
// Waves are independent: each takes its own tickets, uses its own slice of LDS and never
// meets a workgroup barrier.  The backward does the same from the last row to the first for
// dx = dy + a[next]*dx[next], keeps the forward values y (float32, from the states the forward
// pass saved) in registers and forms dA[m] = a[m] * <dx[m], y[m-1]> on the way.
#pragma once
#include "ema_chain_kernels.h"

namespace ema {

#ifdef EMA_TIMING
#define EMA_WSTAMP(slot)                                                                      \
  do {                                                                                        \
    if (lane == 0 && g_ema_timing) g_ema_timing[(int64_t)cur * 8 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define EMA_WSTAMP(slot) \
  do {                   \
  } while (0)
#endif

constexpr int kLaneRows = 32;  // rows per lane; 4 row groups of 16 lanes make the 128-row tile

template <typename T, int CPL>
struct WaveCfg {
  static constexpr int BN = 16 * CPL;                   // columns of a wave tile
  static constexpr int NW = CPL * (int)sizeof(T) / 4;   // 32-bit words of one lane's row
  static constexpr int KPL = (BN + 63) / 64;            // published columns per lane
  static constexpr int LDS_FLOATS = 128 + 8 * BN;       // a[128], forward and reverse group states
  static_assert(NW == 2 || NW == 4, "a lane's row is 8 or 16 bytes");
};

template <int NW>
struct RowWords {
  unsigned w[NW];
};

template <int NW>
__device__ __forceinline__ RowWords<NW> row_load(const void* p) {
  RowWords<NW> r;
  if constexpr (NW == 4) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    r.w[0] = v.x, r.w[1] = v.y, r.w[2] = v.z, r.w[3] = v.w;
  } else {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    r.w[0] = v.x, r.w[1] = v.y;
  }
  return r;
}
template <int NW>
__device__ __forceinline__ void row_store(void* p, const RowWords<NW>& r) {
  if constexpr (NW == 4) *reinterpret_cast<uint4*>(p) = make_uint4(r.w[0], r.w[1], r.w[2], r.w[3]);
  else *reinterpret_cast<uint2*>(p) = make_uint2(r.w[0], r.w[1]);
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

// Orders the LDS traffic of the lanes of one wave (no workgroup barrier: a wave's LDS
// instructions execute in order, the fences only stop the compiler from moving them).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sum over the 16 lanes of a row group, returned in every lane of the group.
__device__ __forceinline__ float group16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124 /* row_ror:4 */, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4e /* quad_perm:[2,3,0,1] */, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xb1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, false));
  return v;
}

// Loads the tile's 32 rows of this lane.  g points at (first row of the tile, first column of
// the tile) of the sequence; rows at or past `limit` and columns at or past the end read as 0.
template <typename T, int CPL>
__device__ __forceinline__ void wave_load_rows(RowWords<WaveCfg<T, CPL>::NW>* rows, const T* __restrict__ g,
                                               int64_t sl, int limit, bool cok, int lane) {
  constexpr int NW = WaveCfg<T, CPL>::NW;
  const int r0 = kLaneRows * (lane >> 4);
  const unsigned off = (unsigned)r0 * (unsigned)sl + (unsigned)(lane & 15) * CPL;
  if (limit == kTileRows && __all(cok)) {
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i) rows[i] = row_load<NW>(g + (int64_t)i * sl + off);
  } else {
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i)
      rows[i] = (r0 + i < limit && cok) ? row_load<NW>(g + (int64_t)i * sl + off) : row_zero<NW>();
  }
}

// Per-row decay factors a[m] = exp(min(A[m], 0)) of the tile into LDS (1 past the end of the
// sequence), and the total decay of each 32-row group as uniform values.
__device__ __forceinline__ void wave_decays(float* aT, float* D, const float* __restrict__ A,
                                            int64_t a_sl, int limit, int lane) {
  const float A0 = lane < limit ? fminf(A[(int64_t)lane * a_sl], 0.f) : 0.f;
  const float A1 = lane + 64 < limit ? fminf(A[(int64_t)(lane + 64) * a_sl], 0.f) : 0.f;
  aT[lane] = __expf(A0);
  aT[lane + 64] = __expf(A1);
  const float s0 = wave_inclusive_scan(A0), s1 = wave_inclusive_scan(A1);
  const float h0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s0), 31));
  const float t0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s0), 63));
  const float h1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s1), 31));
  const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s1), 63));
  D[0] = __expf(h0);
  D[1] = __expf(t0 - h0);
  D[2] = __expf(h1);
  D[3] = __expf(t1 - h1);
}

// chain_look for the KPL columns lane + 64*j of one lane at once: the words of one earlier
// tile are requested together, so the walk costs one round trip per tile, not per column.
template <bool REV, int BN, int KPL>
__device__ __forceinline__ void chain_look_cols(float* carry, const u64* status,
                                                const float* __restrict__ cs_n, int c, int C, int lane,
                                                unsigned* err) {
  float scale = 1.f;
  bool open[KPL];
#pragma unroll
  for (int q = 0; q < KPL; ++q) carry[q] = 0.f, open[q] = lane + 64 * q < BN;
  for (int j = REV ? c + 1 : c - 1; REV ? j < C : j >= 0; j += REV ? 1 : -1) {
    u64 w[KPL];
#pragma unroll
    for (int q = 0; q < KPL; ++q)
      w[q] = open[q] ? __hip_atomic_load(status + (int64_t)j * BN + lane + 64 * q, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT)
                     : 0ull;
    bool any = false;
#pragma unroll
    for (int q = 0; q < KPL; ++q) {
      if (!open[q]) continue;
      unsigned f = (unsigned)(w[q] >> 32);
      float v = __uint_as_float((unsigned)w[q]);
      if (!f) f = chain_wait(status + (int64_t)j * BN + lane + 64 * q, &v, err);
      carry[q] = fmaf(scale, v, carry[q]);
      if (f == kFlagPrefix) open[q] = false;
      any |= open[q];
    }
    if (!any) break;
    scale *= __expf(fminf(cs_n[(int64_t)j * kTileRows + kTileRows - 1], 0.f));
  }
}

// a[m] of rows i .. i+3 of row group grp.
__device__ __forceinline__ void wave_a4(float* a, const float* aT, int grp, int i) {
  const float4 v = *reinterpret_cast<const float4*>(&aT[kLaneRows * grp + i]);
  a[0] = v.x, a[1] = v.y, a[2] = v.z, a[3] = v.w;
}

// Makes the registers of a tile opaque to the optimiser, so that values derived from them in
// one pass (the float32 conversions) are formed again in the next pass instead of being kept.
template <int NW>
__device__ __forceinline__ void rows_opaque(RowWords<NW>* rows) {
#pragma unroll
  for (int i = 0; i < kLaneRows; ++i)
#pragma unroll
    for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(rows[i].w[k]));
}

// ------------------------------------------------------------------------------------
// Forward.  Writes y, prev[n,c,:] (state entering each 128-row chunk), optionally a copy at
// a coarser chunking and the final state.  status: N*ntiles*C*BN zeroed words; counters[0]
// ticket, counters[3] error word.
// ------------------------------------------------------------------------------------
template <typename T, int CPL, int NWAVES, int MINW>
__global__ __launch_bounds__(64 * NWAVES, MINW) void fwd_wave_kernel(
    const T* __restrict__ x, SeqStrides sx, const float* __restrict__ A, SeqStrides sa,
    const float* __restrict__ cs, T* __restrict__ y, SeqStrides sy, float* __restrict__ prev,
    float* __restrict__ prev_coarse, int ratio, float* __restrict__ final_state,
    u64* __restrict__ status, unsigned* __restrict__ counters, int nh, int L, int Tdim, int C,
    int ntiles, int cols, int total) {
  using W = WaveCfg<T, CPL>;
  constexpr int BN = W::BN, NW = W::NW;
  __shared__ __attribute__((aligned(16))) float lds[NWAVES][W::LDS_FLOATS];
  float* aT = lds[threadIdx.x >> 6];
  float* sS = aT + 128;  // [4][BN] group states
  const int lane = threadIdx.x & 63;
  const int grp = lane >> 4, lc = lane & 15;
  unsigned* err = counters + 3;

  // One ticket per workgroup and round: its waves take NWAVES consecutive tiles (adjacent
  // column tiles of the same rows).  The ticket after is fetched while the tiles are processed.
  __shared__ int s_ticket[2];
  if (threadIdx.x == 0) s_ticket[0] = (int)atomicAdd(counters, 1u);
  __syncthreads();
  int wg_cur = s_ticket[0], slot = 1;
  while (wg_cur * NWAVES < total) {
    if (threadIdx.x == 0) s_ticket[slot] = (int)atomicAdd(counters, 1u);
    const int cur = wg_cur * NWAVES + (threadIdx.x >> 6);
    if (cur < total) {
    const ChainTile t = chain_decode<false, BN>(cur, cols, ntiles, C, nh, L);
    const bool cok = t.col0 + lc * CPL < Tdim;
    EMA_WSTAMP(0);
    RowWords<NW> rows[kLaneRows];
    wave_load_rows<T, CPL>(rows, x + (int64_t)t.b * sx.sb + (int64_t)t.h * sx.sh +
                                     (int64_t)t.c * kTileRows * sx.sl + t.col0,
                           sx.sl, t.limit, cok, lane);
    float D[4];
    wave_decays(aT, D, A + (int64_t)t.b * sa.sb + (int64_t)t.h * sa.sh + (int64_t)t.c * kTileRows * sa.sl,
                sa.sl, t.limit, lane);
    wave_lds_sync();

    // 1. local pass
    float s[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
    for (int i = 0; i < kLaneRows; i += 4) {
      float a[4];
      wave_a4(a, aT, grp, i);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = fmaf(a[q], s[e], row_get<T, NW>(rows[i + q], e));
    }
#pragma unroll
    for (int e = 0; e < CPL; ++e) sS[grp * BN + lc * CPL + e] = s[e];
    rows_opaque<NW>(rows);
    wave_lds_sync();
    EMA_WSTAMP(1);

    // 2. tile aggregate, look-back, states entering the row groups
    u64* st = status + (int64_t)t.col_id * C * BN;
    const float dec = (D[0] * D[1]) * (D[2] * D[3]);
    float S0[W::KPL], S1[W::KPL], S2[W::KPL], loc[W::KPL], p_in[W::KPL];
#pragma unroll
    for (int j = 0; j < W::KPL; ++j) {
      const int k = lane + 64 * j;
      if (k < BN) {
        S0[j] = sS[k], S1[j] = sS[BN + k], S2[j] = sS[2 * BN + k];
        loc[j] = fmaf(D[3], fmaf(D[2], fmaf(D[1], S0[j], S1[j]), S2[j]), sS[3 * BN + k]);
        if (t.c > 0) chain_publish(st + (int64_t)t.c * BN + k, kFlagAggregate, loc[j]);
      }
    }
    EMA_WSTAMP(2);
    chain_look_cols<false, BN, W::KPL>(p_in, st, cs + (int64_t)t.n * C * kTileRows, t.c, C, lane, err);
#pragma unroll
    for (int j = 0; j < W::KPL; ++j) {
      const int k = lane + 64 * j;
      if (k < BN) {
        const float p_out = fmaf(dec, p_in[j], loc[j]);
        chain_publish(st + (int64_t)t.c * BN + k, kFlagPrefix, p_out);
        if (t.col0 + k < Tdim) {
          prev[(int64_t)t.chunk_id * Tdim + t.col0 + k] = p_in[j];
          if (prev_coarse && t.c % ratio == 0)
            prev_coarse[((int64_t)t.n * ((C + ratio - 1) / ratio) + t.c / ratio) * Tdim + t.col0 + k] = p_in[j];
          if (t.c == C - 1) final_state[(int64_t)t.n * Tdim + t.col0 + k] = p_out;
        }
        const float E1 = fmaf(D[0], p_in[j], S0[j]), E2 = fmaf(D[1], E1, S1[j]), E3 = fmaf(D[2], E2, S2[j]);
        sS[k] = p_in[j], sS[BN + k] = E1, sS[2 * BN + k] = E2, sS[3 * BN + k] = E3;
      }
    }
    wave_lds_sync();

    EMA_WSTAMP(3);
    // 3. final pass from the true state
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = sS[grp * BN + lc * CPL + e];
    {
      T* g = y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl + t.col0;
      const int r0 = kLaneRows * grp;
      const unsigned off = (unsigned)r0 * (unsigned)sy.sl + (unsigned)lc * CPL;
#pragma unroll
      for (int i = 0; i < kLaneRows; i += 4) {
        float a[4];
        wave_a4(a, aT, grp, i);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int e = 0; e < CPL; ++e) s[e] = fmaf(a[q], s[e], row_get<T, NW>(rows[i + q], e));
          if (r0 + i + q < t.limit && cok)
            row_store<NW>(g + (int64_t)(i + q) * sy.sl + off, row_pack<T, CPL, NW>(s));
        }
      }
    }
    wave_lds_sync();  // the next tile overwrites this wave's LDS
    EMA_WSTAMP(4);
    }
    __syncthreads();
    wg_cur = s_ticket[slot];
    slot ^= 1;
  }
}

// ------------------------------------------------------------------------------------
// Backward.  prev[n,c,:] (states entering each 128-row chunk, from the forward) is an input;
// the reverse state entering each tile from the rows after it, H = a[next row] * dx[next row],
// comes from the chained scan over dy, last chunk first.  Writes dx, optionally y, and the
// column partials part[(chunk*ntiles + ctile)*128 + m] = a[m] * <dx[m], y[m-1]> over the
// tile's columns.  counters[1] ticket, counters[3] error word.
// ------------------------------------------------------------------------------------
template <typename T, int CPL, int NWAVES, int MINW, bool WRITE_Y>
__global__ __launch_bounds__(64 * NWAVES, MINW) void bwd_wave_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ A, SeqStrides sa, const float* __restrict__ cs,
    const float* __restrict__ prev, T* __restrict__ dx, SeqStrides sdx, T* __restrict__ y,
    SeqStrides sy, float* __restrict__ part, u64* __restrict__ status,
    unsigned* __restrict__ counters, int nh, int L, int Tdim, int C, int ntiles, int cols, int total) {
  using W = WaveCfg<T, CPL>;
  constexpr int BN = W::BN, NW = W::NW;
  __shared__ __attribute__((aligned(16))) float lds[NWAVES][W::LDS_FLOATS];
  float* aT = lds[threadIdx.x >> 6];
  float* sS = aT + 128;       // [4][BN] forward group states
  float* sR = sS + 4 * BN;    // [4][BN] reverse group states
  const int lane = threadIdx.x & 63;
  const int grp = lane >> 4, lc = lane & 15;
  unsigned* err = counters + 3;

  // One ticket per workgroup and round: its waves take NWAVES consecutive tiles (adjacent
  // column tiles of the same rows).  The ticket after is fetched while the tiles are processed.
  __shared__ int s_ticket[2];
  if (threadIdx.x == 0) s_ticket[0] = (int)atomicAdd(counters + 1, 1u);
  __syncthreads();
  int wg_cur = s_ticket[0], slot = 1;
  while (wg_cur * NWAVES < total) {
    if (threadIdx.x == 0) s_ticket[slot] = (int)atomicAdd(counters + 1, 1u);
    const int cur = wg_cur * NWAVES + (threadIdx.x >> 6);
    if (cur < total) {
    const ChainTile t = chain_decode<true, BN>(cur, cols, ntiles, C, nh, L);
    const bool cok = t.col0 + lc * CPL < Tdim;
    EMA_WSTAMP(0);
    RowWords<NW> dr[kLaneRows], xr[kLaneRows];
    wave_load_rows<T, CPL>(dr, dy + (int64_t)t.b * sd.sb + (int64_t)t.h * sd.sh +
                                   (int64_t)t.c * kTileRows * sd.sl + t.col0,
                           sd.sl, t.limit, cok, lane);
    wave_load_rows<T, CPL>(xr, x + (int64_t)t.b * sx.sb + (int64_t)t.h * sx.sh +
                                   (int64_t)t.c * kTileRows * sx.sl + t.col0,
                           sx.sl, t.limit, cok, lane);
    float p_in[W::KPL];
#pragma unroll
    for (int j = 0; j < W::KPL; ++j) {
      const int k = lane + 64 * j;
      p_in[j] = (k < BN && t.col0 + k < Tdim) ? prev[(int64_t)t.chunk_id * Tdim + t.col0 + k] : 0.f;
    }
    float D[4];
    wave_decays(aT, D, A + (int64_t)t.b * sa.sb + (int64_t)t.h * sa.sh + (int64_t)t.c * kTileRows * sa.sl,
                sa.sl, t.limit, lane);
    wave_lds_sync();

    // 1a. local reverse pass over dy, r = a[i] * dx_local[i]; at the end the state that the
    // group hands to the rows before it
    float r[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) r[e] = 0.f;
#pragma unroll
    for (int i = kLaneRows - 4; i >= 0; i -= 4) {
      float a[4];
      wave_a4(a, aT, grp, i);
#pragma unroll
      for (int q = 3; q >= 0; --q)
#pragma unroll
        for (int e = 0; e < CPL; ++e) r[e] = a[q] * (row_get<T, NW>(dr[i + q], e) + r[e]);
    }
#pragma unroll
    for (int e = 0; e < CPL; ++e) sR[grp * BN + lc * CPL + e] = r[e];
    rows_opaque<NW>(dr);
    // 1b. local forward pass over x
    float s[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
    for (int i = 0; i < kLaneRows; i += 4) {
      float a[4];
      wave_a4(a, aT, grp, i);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = fmaf(a[q], s[e], row_get<T, NW>(xr[i + q], e));
    }
#pragma unroll
    for (int e = 0; e < CPL; ++e) sS[grp * BN + lc * CPL + e] = s[e];
    rows_opaque<NW>(xr);
    wave_lds_sync();
    EMA_WSTAMP(1);

    // 2a. publish the reverse aggregate; forward states entering the row groups
    u64* st = status + (int64_t)t.col_id * C * BN;
    float loc[W::KPL], R1[W::KPL], R2[W::KPL], R3[W::KPL];
#pragma unroll
    for (int j = 0; j < W::KPL; ++j) {
      const int k = lane + 64 * j;
      if (k < BN) {
        const float R0 = sR[k];
        R1[j] = sR[BN + k], R2[j] = sR[2 * BN + k], R3[j] = sR[3 * BN + k];
        loc[j] = fmaf(D[0], fmaf(D[1], fmaf(D[2], R3[j], R2[j]), R1[j]), R0);
        if (t.c < C - 1) chain_publish(st + (int64_t)t.c * BN + k, kFlagAggregate, loc[j]);
        const float S0 = sS[k], S1 = sS[BN + k], S2 = sS[2 * BN + k];
        const float E1 = fmaf(D[0], p_in[j], S0), E2 = fmaf(D[1], E1, S1), E3 = fmaf(D[2], E2, S2);
        sS[k] = p_in[j], sS[BN + k] = E1, sS[2 * BN + k] = E2, sS[3 * BN + k] = E3;
      }
    }
    wave_lds_sync();

    // 1c. forward values y from the true state (kept in float32 for the dots)
    float E[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) E[e] = sS[grp * BN + lc * CPL + e];
    float yv[kLaneRows][CPL];
    {
      const int r0 = kLaneRows * grp;
      T* g = WRITE_Y ? y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl + t.col0
                     : nullptr;
      const unsigned off = (unsigned)r0 * (unsigned)sy.sl + (unsigned)lc * CPL;
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = E[e];
#pragma unroll
      for (int i = 0; i < kLaneRows; i += 4) {
        float a[4];
        wave_a4(a, aT, grp, i);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int e = 0; e < CPL; ++e) {
            s[e] = fmaf(a[q], s[e], row_get<T, NW>(xr[i + q], e));
            yv[i + q][e] = s[e];
          }
          if (WRITE_Y && r0 + i + q < t.limit && cok)
            row_store<NW>(g + (int64_t)(i + q) * sy.sl + off, row_pack<T, CPL, NW>(s));
        }
      }
    }

    EMA_WSTAMP(2);
    // 2b. look-back for the reverse state, states entering the row groups from the right
    {
      const float dec = (D[0] * D[1]) * (D[2] * D[3]);
      float h_in[W::KPL];
      chain_look_cols<true, BN, W::KPL>(h_in, st, cs + (int64_t)t.n * C * kTileRows, t.c, C, lane, err);
#pragma unroll
      for (int j = 0; j < W::KPL; ++j) {
        const int k = lane + 64 * j;
        if (k < BN) {
          chain_publish(st + (int64_t)t.c * BN + k, kFlagPrefix, fmaf(dec, h_in[j], loc[j]));
          const float G2 = fmaf(D[3], h_in[j], R3[j]), G1 = fmaf(D[2], G2, R2[j]), G0 = fmaf(D[1], G1, R1[j]);
          sR[k] = G0, sR[BN + k] = G1, sR[2 * BN + k] = G2, sR[3 * BN + k] = h_in[j];
        }
      }
    }
    wave_lds_sync();

    EMA_WSTAMP(3);
    // 3. final reverse pass: dx, and the dots with the row before
    {
      const int r0 = kLaneRows * grp;
      T* g = dx + (int64_t)t.b * sdx.sb + (int64_t)t.h * sdx.sh + (int64_t)t.c * kTileRows * sdx.sl + t.col0;
      const unsigned off = (unsigned)r0 * (unsigned)sdx.sl + (unsigned)lc * CPL;
      float dA0 = 0.f, dA1 = 0.f;  // this lane reports rows lc and lc + 16 of its group
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = sR[grp * BN + lc * CPL + e];
#pragma unroll
      for (int i4 = kLaneRows - 4; i4 >= 0; i4 -= 4) {
        float a[4];
        wave_a4(a, aT, grp, i4);
#pragma unroll
        for (int q = 3; q >= 0; --q) {
          const int i = i4 + q;
          float dot = 0.f;
#pragma unroll
          for (int e = 0; e < CPL; ++e) {
            // r holds a[i+1] * dx[i+1] on entry (the carried state for the last row)
            const float d = row_get<T, NW>(dr[i], e) + r[e];
            dot = fmaf(d, i > 0 ? yv[i - 1][e] : E[e], dot);
            r[e] = d;
          }
          if (r0 + i < t.limit && cok) row_store<NW>(g + (int64_t)i * sdx.sl + off, row_pack<T, CPL, NW>(r));
#pragma unroll
          for (int e = 0; e < CPL; ++e) r[e] *= a[q];
          dot = a[q] * group16_sum(dot);
          if ((i & 15) == lc) {
            if (i < 16) dA0 = dot;
            else dA1 = dot;
          }
        }
      }
      float* pp = part + ((int64_t)t.chunk_id * ntiles + t.ctile) * kTileRows + r0;
      pp[lc] = r0 + lc < t.limit ? dA0 : 0.f;
      pp[lc + 16] = r0 + lc + 16 < t.limit ? dA1 : 0.f;
    }
    wave_lds_sync();
    EMA_WSTAMP(4);
    }
    __syncthreads();
    wg_cur = s_ticket[slot];
    slot ^= 1;
  }
}

}  // namespace ema
