// The intra-chunk log-decay gradient (stage B6 on its own) without a Q x Q product.
//
// Where the cumsum cs never rises inside a chunk, exp(min(cs[m] - cs[k], 0)) = a[k+1] * ... * a[m]
// with a[j] = exp(cs[j] - cs[j-1]), and the sum of the weighted triangle over the rows m >= j and the
// columns k < j factors:
//
//   ddA[j] = a[j] * < r[j], y[j-1] >,   y[j] = a[j] * y[j-1] + x[j]        (from 0 at the chunk's start)
//                                       r[j] = dy[j] + a[j+1] * r[j+1]     (from 0 at the chunk's end)
//
// two scans local to the chunk and one dot per row: time and traffic do not grow with Q.  A chunk in
// which cs rises somewhere is flagged (steep[chunk] = 1) and left to the kernel that forms the
// product, which takes the minimum pair by pair.
//
// A workgroup owns all rows of a chunk for BN columns and keeps its x rows in registers: wave g owns
// the RPL rows 128*t + RPL*g .. of each of the chunk's KT sub-tiles of 128 rows (lane l the CPL
// adjacent columns CPL*l ..), as the single-pass kernels do.  Per chunk:
//   1. the local forward passes of all sub-tiles, in the order their rows arrive (last first);
//   2. sub-tiles from the last to the first: local reverse pass over dy; one thread per column chains
//      the reverse group states (the state entering the sub-tile from the rows after it stays in that
//      thread's register from one sub-tile to the next), and, once per chunk, one thread per column
//      chains the forward group states through all sub-tiles; then the forward values from the true
//      state and the reverse pass with the dots.
// Behind the last use of a row the row that takes its registers next is requested: the dy row of
// the sub-tile before, the x row of the same sub-tile of the workgroup's next chunk.
#pragma once
#include "ema_tile_kernels.h"

namespace ema {

// The rows of a chunk are read through a buffer descriptor over the chunk's valid rows of one column
// tile: a load costs one 32-bit offset (the lane's columns plus the row), rows at or past the limit
// fall outside the descriptor's range and read as 0, and a lane whose columns lie past the tensor
// carries an offset outside every range.
constexpr unsigned kFlatNoColumn = 0x80000000u;
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t flat_rows_desc(const T* base, int64_t sl, int limit, int ncols) {
  const int bytes = limit > 0 ? (int)(((int64_t)(limit - 1) * sl + ncols) * (int64_t)sizeof(T)) : 0;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, bytes, 0x00020000);
}
typedef unsigned flat_u2 __attribute__((ext_vector_type(2)));
typedef unsigned flat_u4 __attribute__((ext_vector_type(4)));
template <int NW>
__device__ __forceinline__ RowWords<NW> flat_load_row(__amdgpu_buffer_rsrc_t desc, unsigned voff) {
  constexpr int kNonTemporal = 2;
  RowWords<NW> r;
  if constexpr (NW == 4) {
    const flat_u4 v = __builtin_bit_cast(flat_u4, __builtin_amdgcn_raw_buffer_load_b128(desc, voff, 0, kNonTemporal));
    r.w[0] = v[0], r.w[1] = v[1], r.w[2] = v[2], r.w[3] = v[3];
  } else if constexpr (NW == 2) {
    const flat_u2 v = __builtin_bit_cast(flat_u2, __builtin_amdgcn_raw_buffer_load_b64(desc, voff, 0, kNonTemporal));
    r.w[0] = v[0], r.w[1] = v[1];
  } else {
    r.w[0] = __builtin_amdgcn_raw_buffer_load_b32(desc, voff, 0, kNonTemporal);
  }
  return r;
}

template <typename T, int CPL, int RPL, int KT>
struct FlatCfg {
  using W = TileCfg<T, CPL, RPL>;
  static constexpr int kStateFloats = KT * W::NG * W::BN;  // forward group states of every sub-tile
  static constexpr int kRevFloats = 2 * W::NG * W::BN;     // reverse group states, double-buffered
  static constexpr int kDecayFloats = KT * W::NG;
  static constexpr int smem_bytes = (kStateFloats + kRevFloats + kDecayFloats) * (int)sizeof(float);
};

// part[(chunk*ntiles + ctile)*Q + q]: the dot of row q over the columns of tile ctile, times a[q].
// steep[chunk]: 1 where the factored form does not hold (written by the workgroup of column tile 0).
template <typename T, int CPL, int RPL, int KT>
__global__ __launch_bounds__(64 * (kTileRows / RPL), 1) void da_flat_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ cs, float* __restrict__ part, int* __restrict__ steep, int nh, int L, int Tdim,
    int Q, int C, int ntiles, int total) {
  using W = TileCfg<T, CPL, RPL>;
  using F = FlatCfg<T, CPL, RPL, KT>;
  constexpr int BN = W::BN, NW = W::NW, NG = W::NG, NT = W::NT;
  static_assert(2 * BN <= NT, "one thread per column and direction");
  extern __shared__ __attribute__((aligned(16))) float flat_smem[];
  float (*sS)[NG][BN] = reinterpret_cast<float (*)[NG][BN]>(flat_smem);
  float (*sR)[NG][BN] = reinterpret_cast<float (*)[NG][BN]>(flat_smem + F::kStateFloats);
  float (*sD)[NG] = reinterpret_cast<float (*)[NG]>(flat_smem + F::kStateFloats + F::kRevFloats);
  const int lane = threadIdx.x & 63;
  const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const unsigned off = (unsigned)lane * CPL;
  const int kf = (int)threadIdx.x - BN;  // column of the threads that chain the forward group states

  struct Item {
    int64_t chunk_id, xbase, dbase;  // element offsets of the chunk's first row at the tile's first column
    int ctile, limit, ncols;
    unsigned voff;  // byte offset of this lane's columns in a row
  };
  auto decode = [&](int w) {
    Item it;
    it.ctile = w % ntiles;
    it.chunk_id = w / ntiles;
    const int64_t n = it.chunk_id / C;
    const int c = (int)(it.chunk_id - n * C);
    const int64_t b = n / nh;
    const int h = (int)(n - b * nh);
    const int col0 = it.ctile * BN;
    it.limit = min(Q, L - c * Q);
    it.ncols = min(BN, Tdim - col0);
    it.voff = lane * CPL < it.ncols ? off * (unsigned)sizeof(T) : kFlatNoColumn;
    it.xbase = b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl + col0;
    it.dbase = b * sd.sb + h * sd.sh + (int64_t)c * Q * sd.sl + col0;
    return it;
  };
  // byte offset of row i of this wave in sub-tile t, for a row pitch of pitch bytes
  auto row_off = [&](int t, int i, unsigned pitch) { return (unsigned)(kTileRows * t + RPL * grp + i) * pitch; };
  // The row pitches in bytes.  Every sub-tile takes them through opaque(), so that the offsets of its
  // rows are formed where they are used and not kept for the whole kernel in scalar registers that
  // are needed for other things.
  const unsigned xpitch = (unsigned)sx.sl * (unsigned)sizeof(T), dpitch = (unsigned)sd.sl * (unsigned)sizeof(T);
  auto opaque = [](unsigned v) {
    asm volatile("" : "+s"(v));
    return v;
  };
  // Lane RPL*t + i: cs[q] - cs[q-1] for row i of this wave in sub-tile t (cs[0] itself for the
  // chunk's first row, 0 for rows at or past the limit).  One register holds the wave's coefficients
  // of the whole chunk; a row's value is read from its lane where it is used.
  static_assert(RPL * KT <= 64, "one lane per row of the wave");
  auto coef_load = [&](const Item& it) {
    const int q = kTileRows * (lane / RPL) + RPL * grp + lane % RPL;
    float raw = 0.f;
    if (lane < RPL * KT && q < it.limit) {
      const float* p = cs + it.chunk_id * Q + q;
      raw = p[0] - (q > 0 ? p[-1] : 0.f);
    }
    return raw;
  };
  auto row_coef = [](float v, int i) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i)); };

  RowWords<NW> xr[KT][RPL], dr[RPL];
  float araw = 0.f;
  int w = blockIdx.x, buf = 0;
  Item it = decode(w < total ? w : 0);
  if (w < total) {
    const __amdgpu_buffer_rsrc_t xd = flat_rows_desc(x + it.xbase, sx.sl, it.limit, it.ncols);
    const __amdgpu_buffer_rsrc_t dd = flat_rows_desc(dy + it.dbase, sd.sl, it.limit, it.ncols);
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
#pragma unroll
      for (int i = 0; i < RPL; ++i) xr[t][i] = flat_load_row<NW>(xd, it.voff + row_off(t, i, xpitch));
      if (t == KT - 1) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) dr[i] = flat_load_row<NW>(dd, it.voff + row_off(t, i, dpitch));
      }
    }
    araw = coef_load(it);
  }
  while (w < total) {
    const int wn = w + (int)gridDim.x;
    const bool more = wn < total;
    const Item nx = decode(more ? wn : 0);
    const __amdgpu_buffer_rsrc_t dd = flat_rows_desc(dy + it.dbase, sd.sl, it.limit, it.ncols);
    const __amdgpu_buffer_rsrc_t xdn = flat_rows_desc(x + nx.xbase, sx.sl, nx.limit, nx.ncols);
    const __amdgpu_buffer_rsrc_t ddn = flat_rows_desc(dy + nx.dbase, sd.sl, nx.limit, nx.ncols);
    // lane RPL*t + i: the decay of row i of this wave in sub-tile t
    const float av = __expf(fminf(araw, 0.f));
    const bool rises = araw > 0.f && kTileRows * (lane / RPL) + RPL * grp + lane % RPL > 0;

    // 1. local forward passes
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
      __builtin_amdgcn_sched_barrier(0);
      float s[CPL], D = 1.f;
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        D *= row_coef(av, RPL * t + i);
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = fmaf(row_coef(av, RPL * t + i), s[e], row_get<T, NW>(xr[t][i], e));
      }
#pragma unroll
      for (int e = 0; e < CPL; ++e) sS[t][grp][lane * CPL + e] = s[e];
      if (lane == 0) sD[t][grp] = D;
      rows_opaque<NW, RPL>(xr[t]);
    }

    float h_in = 0.f;  // chain threads: reverse state entering the sub-tile from the rows after it
    int flagged = 0;
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
      // 2a. local reverse pass over dy: what the group hands to the rows before it
      __builtin_amdgcn_sched_barrier(0);
      float r[CPL];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = 0.f;
#pragma unroll
      for (int i = RPL - 1; i >= 0; --i)
#pragma unroll
        for (int e = 0; e < CPL; ++e) r[e] = row_coef(av, RPL * t + i) * (row_get<T, NW>(dr[i], e) + r[e]);
#pragma unroll
      for (int e = 0; e < CPL; ++e) sR[buf][grp][lane * CPL + e] = r[e];
      rows_opaque<NW, RPL>(dr);
      if (t == KT - 1) flagged = __syncthreads_or(rises ? 1 : 0);
      else __syncthreads();

      // 2b. chains over the row groups
      if (threadIdx.x < BN) {
        const int k = threadIdx.x;
        float rg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) rg[g] = sR[buf][g][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[t][g]);
#pragma unroll
        for (int g = NG - 1; g >= 0; --g) {
          sR[buf][g][k] = h_in;
          h_in = fmaf(dg[g], h_in, rg[g]);
        }
      } else if (t == KT - 1 && kf < BN) {
        float E = 0.f;
#pragma unroll 1
        for (int u = 0; u < KT; ++u) {
          float sg[NG], dg[NG];
#pragma unroll
          for (int g = 0; g < NG; ++g) sg[g] = sS[u][g][kf];
#pragma unroll
          for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[u][g]);
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            sS[u][g][kf] = E;
            E = fmaf(dg[g], E, sg[g]);
          }
        }
      }
      __syncthreads();

      // 2c. reverse pass with the dots, in segments of SEG of the wave's rows so that few forward
      // values are held at a time: for each segment, last first, the forward recurrence runs from the
      // state entering the group to the segment, its values over the segment are kept, and the reverse
      // pass takes the segment's rows.  Behind the last use of a row the row that uses its registers
      // next is requested.
      constexpr int SEG = KT >= 3 ? 2 : 4;
      const unsigned xp = opaque(xpitch), dp = opaque(dpitch);
      float dA = 0.f;  // lane i reports row i of the wave
      // (this lane's number, formed per sub-tile so that the eight comparisons with it are not kept)
      const unsigned me = __builtin_amdgcn_mbcnt_hi(opaque(~0u), __builtin_amdgcn_mbcnt_lo(opaque(~0u), 0u));
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = sR[buf][grp][lane * CPL + e];
#pragma unroll
      for (int i0 = RPL - SEG; i0 >= 0; i0 -= SEG) {
        __builtin_amdgcn_sched_barrier(0);
        float ym[CPL];  // forward value of the row before the segment
#pragma unroll
        for (int e = 0; e < CPL; ++e) ym[e] = sS[t][grp][lane * CPL + e];
#pragma unroll
        for (int i = 0; i < i0; ++i)
#pragma unroll
          for (int e = 0; e < CPL; ++e) ym[e] = fmaf(row_coef(av, RPL * t + i), ym[e], row_get<T, NW>(xr[t][i], e));
        float yv[SEG - 1][CPL];  // forward values of the segment's rows but the last
        {
          float s[CPL];
#pragma unroll
          for (int e = 0; e < CPL; ++e) s[e] = ym[e];
#pragma unroll
          for (int i = 0; i < SEG - 1; ++i)
#pragma unroll
            for (int e = 0; e < CPL; ++e) {
              s[e] = fmaf(row_coef(av, RPL * t + i0 + i), s[e], row_get<T, NW>(xr[t][i0 + i], e));
              yv[i][e] = s[e];
            }
        }
#pragma unroll
        for (int j = SEG - 1; j >= 0; --j) {
          __builtin_amdgcn_sched_barrier(0);
          const int i = i0 + j;
          float dot = 0.f;
#pragma unroll
          for (int e = 0; e < CPL; ++e) {
            const float d = row_get<T, NW>(dr[i], e) + r[e];
            dot = fmaf(d, j > 0 ? yv[j - 1][e] : ym[e], dot);
            r[e] = d * row_coef(av, RPL * t + i);
          }
          if (t > 0) dr[i] = flat_load_row<NW>(dd, it.voff + row_off(t - 1, i, dp));
          else if (more) dr[i] = flat_load_row<NW>(ddn, nx.voff + row_off(KT - 1, i, dp));
          if (more) xr[t][i] = flat_load_row<NW>(xdn, nx.voff + row_off(t, i, xp));
          // the row's dot goes into lane i (rows at or past the limit have dy = 0 and give 0)
          const float total = wave_sum(dot) * row_coef(av, RPL * t + i);
          if (me == (unsigned)i) dA = total;
        }
      }
      {
        // a scalar base and this lane's row as a 32-bit offset, formed here and not kept
        const int q0 = kTileRows * t + RPL * grp;
        float* pb = part + ((it.chunk_id * ntiles + it.ctile) * (int64_t)Q + q0);
        if (me < (unsigned)RPL && q0 + (int)me < Q) pb[me] = dA;
      }
      buf ^= 1;
    }
    if (threadIdx.x == 0 && it.ctile == 0) steep[it.chunk_id] = flagged;
    if (more) {
      araw = coef_load(nx);
    }
    w = wn;
    it = nx;
  }
}

}  // namespace ema
