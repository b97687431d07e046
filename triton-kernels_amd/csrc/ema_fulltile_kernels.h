// Single-pass forward of the EMA scan for problems made of whole tiles (seqlen a multiple of
// 128, dim a multiple of the tile width), which is what the benchmark shapes are.  Same algorithm,
// tile order, chained scan and workspace as fwd_tile_kernel in ema_tile_kernels.h, which stays for
// every other shape; what differs is how a workgroup is organised.  That kernel executes about 360
// vector and 330 scalar instructions per wave and tile, serialises a tile's phases (rows arrive,
// local pass, chain over the row groups, look-back, final pass, stores) with two barriers, and its
// look-back waves also own rows.  Here
//
//   * nothing is predicated (whole tiles), addresses are a scalar base per tile plus one 32-bit
//     lane offset, and the tile a ticket stands for is found with multiplications by
//     precomputed reciprocals instead of divisions;
//   * the coefficients of a wave's 16 rows arrive with one load (lane j takes row j % 16) and a
//     row's decay is read from its lane when needed;
//   * the chain over the row groups, the publishing and the look-back are done by waves of
//     their own that own no rows (one thread per column): their polls never queue behind row
//     loads (a wave's memory operations complete in order);
//   * a workgroup works on two tiles at a time, so that the look-back of one tile runs while the
//     rows of the next are scanned, and requests rows two tiles ahead.
#pragma once
#include "ema_tile_kernels.h"

namespace ema {

constexpr int kFullRowWaves = 8;                       // waves that own rows
constexpr int kFullRpl = kTileRows / kFullRowWaves;    // rows per lane: 16

template <typename T>
struct FullCfg {
  static constexpr int CPL = 8 / (int)sizeof(T);  // columns per lane: a lane's row is 8 bytes
  static constexpr int BN = 64 * CPL;             // columns of a tile
  static constexpr int LOOKW = BN / 64;           // waves that chain, publish and look back
  static constexpr int NT = 64 * (kFullRowWaves + LOOKW);
};

// a compile-time flag passed as a function argument
template <int I>
struct IntC {
  static constexpr int value = I;
};

__device__ __forceinline__ int uniform_int(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
// v of the lane `shift` below within each group of 16 lanes, 1 where there is none
template <int CTRL>
__device__ __forceinline__ float dpp_or_one(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0x3f800000, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// inclusive prefix product over each group of 16 lanes
__device__ __forceinline__ float row16_prefix_product(float v) {
  v *= dpp_or_one<0x111>(v);  // row_shr:1
  v *= dpp_or_one<0x112>(v);  // row_shr:2
  v *= dpp_or_one<0x114>(v);  // row_shr:4
  v *= dpp_or_one<0x118>(v);  // row_shr:8
  return v;
}
// 8 bytes of a row: CPL elements as floats, and back
template <typename T>
__device__ __forceinline__ void row8_unpack(uintx2 w, float* v) {
  if constexpr (sizeof(T) == 4) {
    v[0] = __uint_as_float(w[0]);
    v[1] = __uint_as_float(w[1]);
  } else {
    v[0] = __uint_as_float(w[0] << 16);
    v[1] = __uint_as_float(w[0] & 0xffff0000u);
    v[2] = __uint_as_float(w[1] << 16);
    v[3] = __uint_as_float(w[1] & 0xffff0000u);
  }
}
template <typename T>
__device__ __forceinline__ unsigned long long row8_pack(const float* v) {
  unsigned lo, hi;
  if constexpr (sizeof(T) == 4) {
    lo = __float_as_uint(v[0]);
    hi = __float_as_uint(v[1]);
  } else {
    bf16x2 a, b;
    a[0] = (bf16_t)v[0], a[1] = (bf16_t)v[1];
    b[0] = (bf16_t)v[2], b[1] = (bf16_t)v[3];
    lo = __builtin_bit_cast(unsigned, a);
    hi = __builtin_bit_cast(unsigned, b);
  }
  return ((unsigned long long)hi << 32) | lo;
}
// uniform base + 32-bit lane offset
__device__ __forceinline__ uintx2 row8_load(const char* base, unsigned off) {
  if (kStreamFwdLoad) return __builtin_nontemporal_load(reinterpret_cast<const uintx2*>(base + off));
  return *reinterpret_cast<const uintx2*>(base + off);
}
// written through to device memory (a relaxed store at agent scope): nothing of the output stays
// behind as dirty lines in the L2s for the end of the kernel to write back
__device__ __forceinline__ void row8_store(char* base, unsigned off, unsigned long long v) {
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(base + off), v, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

struct FullFwdArgs {
  const char* x;
  char* y;
  const float* A;
  float* prev;         // (N, C, T) state entering each 128-row tile
  float* prev_coarse;  // may be null: the same at a chunking `ratio` times coarser
  float* final_state;  // may be null
  const float* init;   // may be null
  ChainHeader* hdr;
  u64* decw;
  u64* status;
  long long x_sb, x_sl, x_sh, y_sb, y_sl, y_sh;  // bytes
  long long a_sb, a_sl, a_sh;                    // elements
  int ratio, nh, Tdim, C, ntiles, cols, total;
  TileOrder ord;
};

// Per-row coefficients of a row wave, one row per lane (lane j holds row j % 16 of the wave).
//   keep: factor of the state;  gain: factor of x (1 in the log-decay form);
//   reset: probability form only, the state is dropped at this row.
template <bool XP>
struct RowCoef {
  float keep, gain;
  __device__ __forceinline__ void set(float raw) {
    if (XP) {
      gain = fabsf(raw);
      keep = coef_resets(raw) ? 0.f : 1.f - raw;
    } else {
      keep = __expf(fminf(raw, 0.f));
      gain = 1.f;
    }
  }
};

// ------------------------------------------------------------------------------------
// Forward.  Waves 0 .. LOOKW-1 own a column per thread (chain waves), waves LOOKW .. own 16 rows
// each (row waves).  A workgroup works on two tiles at a time, one barrier per tile:
//
//   row waves, step j:    local pass of tile j (group results to LDS) | barrier |
//                         final pass of tile j-1 from the state the chain waves left in LDS, stores |
//                         request the rows of tile j+2 into the registers tile j-1 has freed
//   chain waves, step j:  | barrier | chain over the row groups of tile j, publish, look back,
//                         states entering the row groups to LDS, publish the prefix
//
// so the look-back of a tile has a whole step to complete before anybody waits for it, and the
// rows of a tile are requested two steps before they are used (three register sets of packed
// rows; the final pass runs the recurrence again from the true state, which costs conversions
// but no registers, and gives the values of the sequential recurrence in float32).
// ------------------------------------------------------------------------------------
template <typename T, bool XP>
__global__ __launch_bounds__(FullCfg<T>::NT) void fwd_fulltile_kernel(const FullFwdArgs p) {
  using F = FullCfg<T>;
  constexpr int CPL = F::CPL, BN = F::BN, LOOKW = F::LOOKW, NG = kFullRowWaves, RPL = kFullRpl;
  __shared__ __attribute__((aligned(16))) float sS[2][NG][BN];  // group results, then states entering the groups
  __shared__ __attribute__((aligned(16))) float sD[2][NG];      // total decay of each row group
  __shared__ int s_ticket[4];
  const int lane = threadIdx.x & 63;
  const int wave = uniform_int((int)(threadIdx.x >> 6));
  const ChainCtl ctl = chain_enter(p.hdr);
  const int total = p.total;
  const int Lrows = p.C * kTileRows;

  auto draw = [&]() { return (int)atomicAdd(&p.hdr->ticket, 1u); };
  if (threadIdx.x == 0) {
    s_ticket[0] = draw();
    s_ticket[1] = draw();
    s_ticket[2] = draw();
  }
  __syncthreads();
  // Tickets: step j works on ticket j.  Thread 0 fetches ticket j + 3 during step j (after the
  // barrier) into slot (j + 3) % 4; everybody reads ticket j + 2 right after the barrier of step j.
  int tk0 = uniform_int(s_ticket[0]), tk1 = uniform_int(s_ticket[1]);  // tickets of this step and the next

  if (wave < LOOKW) {
    // ---------------------------------------------------------------- chain waves
    const int k = (int)threadIdx.x;  // column of the tile
    auto words_of = [&](const ChainTile& t) { return p.status + ((long long)t.col_id * p.C) * BN + k; };
    u64 w = 0;  // first look at the predecessor's word, taken a step ahead
    ChainTile t = chain_decode<false, BN>(tk0 < total ? tk0 : 0, p.ord, Lrows);
    if (tk0 < total && t.c > 0) w = chain_peek(words_of(t) + (long long)(t.c - 1) * BN);
    int prev_valid = 0;
    for (int j = 0; tk0 < total || prev_valid; ++j) {
      const int buf = j & 1;
      __syncthreads();  // step j: the row groups' results of tile j are in LDS
      const int tk2 = uniform_int(s_ticket[(j + 2) & 3]);
      int future = 0;
      if (threadIdx.x == 0) future = draw();
      EMA_TSTAMP_DECL;
      EMA_TSTAMP(1);
      EMA_TSTAMP_VALUE(7, (long long)blockIdx.x);
      const int cur = tk0;  // for the stamps
      if (tk0 < total) {
        u64* words = words_of(t);
        float sg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) sg[g] = sS[buf][g][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[buf][g]);
        // loc[g]: state entering group g if nothing entered the tile; dcy[g]: decay of the groups before g
        float loc[NG + 1], dcy[NG + 1];
        loc[0] = 0.f, dcy[0] = 1.f;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          loc[g + 1] = fmaf(dg[g], loc[g], sg[g]);
          dcy[g + 1] = dcy[g] * dg[g];
        }
        EMA_TSTAMP(2);
        float p_in;
        if (t.c > 0) {
          if (k == 0) chain_publish(p.decw + (long long)t.n * p.C + t.c, ctl.epoch, kStateAggregate, dcy[NG]);
          EMA_TSTAMP_VALUE(6, (long long)chain_state(w, ctl.epoch));
          if (chain_state(w, ctl.epoch) == kStatePrefix) {
            p_in = chain_value(w);  // nobody needs this tile's aggregate first
          } else {
            chain_publish(words + (long long)t.c * BN, ctl.epoch, kStateAggregate, loc[NG]);
            ChainLook<false, BN> look;
            look.j = t.c - 1;
            look.w = w;
            p_in = look.finish(words, p.decw + (long long)t.n * p.C, p.C, ctl);
          }
        } else {
          p_in = p.init ? p.init[(long long)t.n * p.Tdim + t.ctile * BN + k] : 0.f;
        }
        EMA_TSTAMP(3);
        const float p_out = fmaf(dcy[NG], p_in, loc[NG]);
        chain_publish(words + (long long)t.c * BN, ctl.epoch, kStatePrefix, p_out);
#pragma unroll
        for (int g = 0; g < NG; ++g) sS[buf][g][k] = fmaf(dcy[g], p_in, loc[g]);
        const long long col = (long long)t.ctile * BN + k;
        p.prev[((long long)t.n * p.C + t.c) * p.Tdim + col] = p_in;
        if (p.prev_coarse && t.c % p.ratio == 0)
          p.prev_coarse[((long long)t.n * ((p.C + p.ratio - 1) / p.ratio) + t.c / p.ratio) * p.Tdim + col] = p_in;
        if (p.final_state && t.c == p.C - 1) p.final_state[(long long)t.n * p.Tdim + col] = p_out;
        EMA_TSTAMP(4);
      }
      if (threadIdx.x == 0) s_ticket[(j + 3) & 3] = future;
      if (tk0 < total) EMA_TSTAMP_FLUSH;
      prev_valid = tk0 < total;
      tk0 = tk1, tk1 = tk2;
      if (tk0 < total) {
        t = chain_decode<false, BN>(tk0, p.ord, Lrows);
        if (t.c > 0) w = chain_peek(words_of(t) + (long long)(t.c - 1) * BN);  // a step ahead of its use
      }
    }
    if (threadIdx.x == 0) chain_leave(p.hdr, ctl);
    return;
  }

  // -------------------------------------------------------------------------- row waves
  const int rg = wave - LOOKW;
  const unsigned voff = (unsigned)lane * 8u;
  struct RowSet {
    uintx2 pk[RPL];
    float araw;
    int b, h, c, ctile;
  };
  RowSet s0, s1, s2;
  auto request = [&](RowSet& rs, int ticket) {
    const ChainTile t = chain_decode<false, BN>(ticket, p.ord, Lrows);
    rs.b = t.b, rs.h = t.h, rs.c = t.c, rs.ctile = t.ctile;
    const long long row0 = (long long)t.c * kTileRows + RPL * rg;
    rs.araw = p.A[t.b * p.a_sb + t.h * p.a_sh + (row0 + (lane & 15)) * p.a_sl];
    const char* g = p.x + t.b * p.x_sb + t.h * p.x_sh + row0 * p.x_sl + (long long)t.ctile * (BN * (int)sizeof(T));
#pragma unroll
    for (int i = 0; i < RPL; ++i) rs.pk[i] = row8_load(g + i * p.x_sl, voff);
  };
  // the recurrence down the 16 rows of this lane from state s; with STORE the values are written out
  auto sweep = [&](const RowSet& rs, float* s, auto store) {
    RowCoef<XP> cf;
    cf.set(rs.araw);
    char* g = p.y + rs.b * p.y_sb + rs.h * p.y_sh + ((long long)rs.c * kTileRows + RPL * rg) * p.y_sl +
              (long long)rs.ctile * (BN * (int)sizeof(T));
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      float xv[CPL];
      row8_unpack<T>(rs.pk[i], xv);
      const float ki = lane_value(cf.keep, i);
      if (XP) {
        const float gi = lane_value(cf.gain, i);
#pragma unroll
        for (int e = 0; e < CPL; ++e) {
          const float b0 = ki != 0.f ? s[e] : 0.f;  // keep = 0: a reset, or p = 1
          s[e] = fmaf(gi, xv[e] - b0, b0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = fmaf(ki, s[e], xv[e]);
      }
      if (decltype(store)::value) row8_store(g + i * p.y_sl, voff, row8_pack<T>(s));
    }
    return cf.keep;
  };
  auto local_pass = [&](const RowSet& rs, int buf) {
    float s[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = 0.f;
    const float keep = sweep(rs, s, IntC<0>{});
    if constexpr (CPL == 4) *reinterpret_cast<float4*>(&sS[buf][rg][lane * 4]) = make_float4(s[0], s[1], s[2], s[3]);
    else *reinterpret_cast<float2*>(&sS[buf][rg][lane * 2]) = make_float2(s[0], s[1]);
    const float P = row16_prefix_product(keep);
    if (lane == 15) sD[buf][rg] = P;
  };
  auto final_pass = [&](const RowSet& rs, int buf) {
    float s[CPL];
    if constexpr (CPL == 4) {
      const float4 e4 = *reinterpret_cast<const float4*>(&sS[buf][rg][lane * 4]);
      s[0] = e4.x, s[1] = e4.y, s[2] = e4.z, s[3] = e4.w;
    } else {
      const float2 e2 = *reinterpret_cast<const float2*>(&sS[buf][rg][lane * 2]);
      s[0] = e2.x, s[1] = e2.y;
    }
    sweep(rs, s, IntC<1>{});
  };
  if (tk0 < total) request(s0, tk0);
  if (tk1 < total) request(s1, tk1);
  int j = 0, prev_valid = 0;
  // one step: rl holds the tile of this step, rf that of the step before, whose registers then
  // receive the tile two steps ahead
  auto step = [&](RowSet& rl, RowSet& rf) {
    const int buf = j & 1;
    EMA_TSTAMP_DECL;
    const int cur = tk0;  // for the stamps
    EMA_TSTAMP_T(64 * LOOKW, 0);
    if (tk0 < total) local_pass(rl, buf);
    EMA_TSTAMP_T(64 * LOOKW, 1);
    __syncthreads();  // step j
    const int tk2 = uniform_int(s_ticket[(j + 2) & 3]);
    EMA_TSTAMP_T(64 * LOOKW, 2);
    if (prev_valid) final_pass(rf, buf ^ 1);
    EMA_TSTAMP_T(64 * LOOKW, 3);
    if (tk2 < total) request(rf, tk2);
    EMA_TSTAMP_T(64 * LOOKW, 4);
    if (tk0 < total) EMA_TSTAMP_FLUSH_T(64 * LOOKW, 8);
    prev_valid = tk0 < total;
    tk0 = tk1, tk1 = tk2;
    ++j;
  };
  for (;;) {
    if (!(tk0 < total || prev_valid)) break;
    step(s0, s2);
    if (!(tk0 < total || prev_valid)) break;
    step(s1, s0);
    if (!(tk0 < total || prev_valid)) break;
    step(s2, s1);
  }
}

}  // namespace ema
