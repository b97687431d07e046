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
// Behind the last use of an x row the row that takes its registers next is requested: the same row
// of the same sub-tile of the workgroup's next chunk, a whole chunk ahead.  The dy rows have no
// registers to wait in: every wave copies the rows of the sub-tile before straight from global memory
// into a place of its own in LDS while it works on this one, and moves them to registers when it gets
// there.
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

// 64 lanes x 16 bytes from global memory into LDS without passing through registers: lane l's piece, at
// base + lane_offset bytes, lands at lds_base + 16 * l.  base and lds_base are the same in every lane.
// The copy counts as a vector-memory load of the wave and completes in order with its other loads.
// First the wave's earlier LDS reads are waited for (they may read the place that is written); m0,
// which carries the LDS address, is put back; the wait states cover a scalar base that vector
// instructions have just written.
typedef __attribute__((address_space(3))) void flat_lds_void_t;
__device__ __forceinline__ void flat_copy16_to_lds(const void* base, unsigned lane_offset, void* lds_base) {
  const unsigned lds = (unsigned)(uintptr_t)(flat_lds_void_t*)lds_base;
  const uint64_t wide = reinterpret_cast<uint64_t>(base);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(wide >> 32));
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)wide);
  base = reinterpret_cast<const void*>(((uint64_t)hi << 32) | (uint64_t)lo);
  unsigned keep;
  asm volatile(
      "s_waitcnt lgkmcnt(0)\n\ts_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(keep)
      : "v"(lane_offset), "s"(base), "s"(lds)
      : "memory");
}
// Waits until at most `newer` of the wave's vector-memory operations are under way: everything but
// the `newer` most recent ones has completed.
template <int NEWER>
__device__ __forceinline__ void flat_wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NEWER) : "memory");
}

template <typename T, int CPL, int RPL, int KT>
struct FlatCfg {
  using W = TileCfg<T, CPL, RPL>;
  static constexpr int kStateFloats = KT * W::NG * W::BN;  // forward group states of every sub-tile
  static constexpr int kRevFloats = W::NG * W::BN;         // reverse group states
  static constexpr int kDecayFloats = KT * W::NG + 4;       // and the flag of a rising cumsum
  static constexpr int kRowBytes = W::BN * (int)sizeof(T);  // a sub-tile's row: 256 or 512 bytes
  static constexpr int kStageBytes = kTileRows * kRowBytes;  // the dy rows of one sub-tile
  static constexpr int smem_bytes = (kStateFloats + kRevFloats + kDecayFloats) * (int)sizeof(float) + kStageBytes;
  static_assert((kStateFloats + kRevFloats + kDecayFloats) % 4 == 0, "the staged rows start at a multiple of 16 bytes");
  static_assert(smem_bytes <= 160 * 1024, "LDS of one compute unit");
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
  float (*sR)[BN] = reinterpret_cast<float (*)[BN]>(flat_smem + F::kStateFloats);
  float (*sD)[NG] = reinterpret_cast<float (*)[NG]>(flat_smem + F::kStateFloats + F::kRevFloats);
  int* const sFlag = reinterpret_cast<int*>(flat_smem + F::kStateFloats + F::kRevFloats + KT * NG);
  const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  // this wave's staged dy rows
  constexpr int ROWB = F::kRowBytes, LPR = ROWB / 16, RPI = 64 / LPR, NCOPY = RPL / RPI;
  static_assert(RPL % RPI == 0, "whole rows per copy");
  char* const stage = reinterpret_cast<char*>(flat_smem + F::kStateFloats + F::kRevFloats + F::kDecayFloats) +
                      grp * (RPL * ROWB);

  auto opaque = [](unsigned v) {
    asm volatile("" : "+s"(v));
    return v;
  };
  if (threadIdx.x == 0) *sFlag = 0;
  __syncthreads();
  // This lane's number, formed anew wherever it is asked for: what is derived from it (LDS addresses,
  // column offsets, comparisons) is then formed where it is used instead of being kept in registers
  // for the whole kernel, and the registers hold rows.
  auto lane_now = [&]() {
    return (int)__builtin_amdgcn_mbcnt_hi(opaque(~0u), __builtin_amdgcn_mbcnt_lo(opaque(~0u), 0u));
  };
  struct Item {
    int64_t chunk_id, xbase, dbase;  // element offsets of the chunk's first row at the tile's first column
    int ctile, limit, ncols;
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
    it.xbase = b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl + col0;
    it.dbase = b * sd.sb + h * sd.sh + (int64_t)c * Q * sd.sl + col0;
    return it;
  };
  // byte offset of lane ln's columns in a row of chunk c (outside every descriptor past the tensor)
  auto col_off = [&](const Item& c, int ln) {
    return ln * CPL < c.ncols ? (unsigned)ln * (unsigned)(CPL * sizeof(T)) : kFlatNoColumn;
  };
  // byte offset of row i of this wave in sub-tile t, for a row pitch of pitch bytes
  auto row_off = [&](int t, int i, unsigned pitch) { return (unsigned)(kTileRows * t + RPL * grp + i) * pitch; };
  // The row pitches in bytes.  Every sub-tile takes them through opaque(), so that the offsets of its
  // rows are formed where they are used and not kept for the whole kernel in scalar registers that
  // are needed for other things.
  const unsigned xpitch = (unsigned)sx.sl * (unsigned)sizeof(T), dpitch = (unsigned)sd.sl * (unsigned)sizeof(T);
  // Lane RPL*t + i: cs[q] - cs[q-1] for row i of this wave in sub-tile t (cs[0] itself for the
  // chunk's first row, 0 for rows at or past the limit).  One register holds the wave's coefficients
  // of the whole chunk; a row's value is read from its lane where it is used.
  static_assert(RPL * KT <= 64, "one lane per row of the wave");
  auto coef_load = [&](const Item& it) {
    const int ln = lane_now();
    const int q = kTileRows * (ln / RPL) + RPL * grp + ln % RPL;
    float raw = 0.f;
    if (ln < RPL * KT && q < it.limit) {
      const float* p = cs + it.chunk_id * Q + q;
      raw = p[0] - (q > 0 ? p[-1] : 0.f);
    }
    return raw;
  };
  auto row_coef = [](float v, int i) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i)); };

  // Requests the dy rows of this wave in sub-tile t of chunk `c` into the wave's place in LDS.  The
  // addresses are clamped into the chunk's valid rows and the tensor's columns (what arrives for a
  // row at or past the limit or a column past the end is dropped when the rows are taken out).
  auto dy_request = [&](const Item& c, int t) {
    const T* base = dy + c.dbase;
    const int me = lane_now();
    const unsigned colb = min((unsigned)(me % LPR) * 16u, (unsigned)c.ncols * (unsigned)sizeof(T) - 16u);
#pragma unroll
    for (int j = 0; j < NCOPY; ++j) {
      const int row = min(kTileRows * t + RPL * grp + RPI * j + me / LPR, c.limit - 1);
      flat_copy16_to_lds(base, (unsigned)row * dpitch + colb, stage + j * 1024);
    }
  };
  // Takes them out (after the wait for the copies).
  auto dy_take = [&](RowWords<NW>* rows, const Item& c, int t) {
    const int nrows = c.limit - (kTileRows * t + RPL * grp);
    const int ln = lane_now();
    const bool cok = ln * CPL < c.ncols;
    const bool full = nrows >= RPL && __all(cok);
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      rows[i] = *reinterpret_cast<const RowWords<NW>*>(stage + i * ROWB + ln * (CPL * (int)sizeof(T)));
      if (!full && !(i < nrows && cok)) rows[i] = row_zero<NW>();
    }
  };

  RowWords<NW> xr[KT][RPL], dr[RPL];
  float araw = 0.f;
  int w = blockIdx.x;
  Item it = decode(w < total ? w : 0);
  if (w < total) {
    const __amdgpu_buffer_rsrc_t xd = flat_rows_desc(x + it.xbase, sx.sl, it.limit, it.ncols);
    dy_request(it, KT - 1);
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
#pragma unroll
      for (int i = 0; i < RPL; ++i) xr[t][i] = flat_load_row<NW>(xd, col_off(it, lane_now()) + row_off(t, i, xpitch));
    }
    araw = coef_load(it);
  }
  while (w < total) {
    const int wn = w + (int)gridDim.x;
    const bool more = wn < total;
    const Item nx = decode(more ? wn : 0);
    const __amdgpu_buffer_rsrc_t xdn = flat_rows_desc(x + nx.xbase, sx.sl, nx.limit, nx.ncols);
    // lane RPL*t + i: the decay of row i of this wave in sub-tile t
    const float av = __expf(fminf(araw, 0.f));
    {
      const int ln = lane_now();
      const bool rises = araw > 0.f && kTileRows * (ln / RPL) + RPL * grp + ln % RPL > 0;
      if (__any(rises) && ln == 0) *sFlag = 1;
    }

    // 1. local forward passes
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
      __builtin_amdgcn_sched_barrier(0);
      float s[CPL], D = 1.f;
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const float ai = row_coef(av, RPL * t + i);
        D *= ai;
#pragma unroll
        for (int e = 0; e < CPL; ++e) s[e] = fmaf(ai, s[e], row_get<T, NW>(xr[t][i], e));
      }
      const int ln = lane_now();
#pragma unroll
      for (int e = 0; e < CPL; ++e) sS[t][grp][ln * CPL + e] = s[e];
      if (ln == 0) sD[t][grp] = D;
      rows_opaque<NW, RPL>(xr[t]);
    }

    float h_in = 0.f;  // chain threads: reverse state entering the sub-tile from the rows after it
#pragma unroll
    for (int t = KT - 1; t >= 0; --t) {
      // The copies of this sub-tile's dy rows were requested one sub-tile ago, and every sub-tile
      // requests the RPL x rows of the next chunk after them (if there is a next chunk; the very first
      // copies are followed by the first chunk's x rows): once at most RPL newer operations are under
      // way they have landed.  Whatever else the wave has issued since only adds to what is waited for.
      __builtin_amdgcn_sched_barrier(0);
      if (t == KT - 1 || more) flat_wait_loads<RPL>();
      else flat_wait_loads<0>();
      dy_take(dr, it, t);
      if (t > 0) dy_request(it, t - 1);
      else if (more) dy_request(nx, KT - 1);
      // 2a. local reverse pass over dy: what the group hands to the rows before it
      __builtin_amdgcn_sched_barrier(0);
      float a[RPL];  // the decays of the wave's rows, in scalar registers for the rest of the sub-tile
#pragma unroll
      for (int i = 0; i < RPL; ++i) a[i] = row_coef(av, RPL * t + i);
      // (u[i] = dy[i] + a[i+1] * u[i+1], one multiply-add per element; the group hands on a[0] * u[0])
      float r[CPL];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = row_get<T, NW>(dr[RPL - 1], e);
#pragma unroll
      for (int i = RPL - 2; i >= 0; --i)
#pragma unroll
        for (int e = 0; e < CPL; ++e) r[e] = fmaf(a[i + 1], r[e], row_get<T, NW>(dr[i], e));
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] *= a[0];
#pragma unroll
      for (int e = 0; e < CPL; ++e) sR[grp][lane_now() * CPL + e] = r[e];
      rows_opaque<NW, RPL>(dr);
      __syncthreads();

      // 2b. chains over the row groups
      constexpr int CW = BN / 64;  // waves with one thread per column
      if (grp < CW) {
        const int k = 64 * grp + lane_now();
        if (t == KT - 1 && k == 0) {
          // the workgroup of column tile 0 reports whether the chunk's cumsum rises anywhere
          if (it.ctile == 0) steep[it.chunk_id] = *sFlag;
          *sFlag = 0;
        }
        float rg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) rg[g] = sR[g][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[t][g]);
#pragma unroll
        for (int g = NG - 1; g >= 0; --g) {
          sR[g][k] = h_in;
          h_in = fmaf(dg[g], h_in, rg[g]);
        }
      } else if (t == KT - 1 && grp < 2 * CW) {
        const int kf = 64 * (grp - CW) + lane_now();
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
      // pass takes the segment's rows.  Behind the last use of an x row the row that uses its registers
      // next is requested (keeping all forward values and requesting the next chunk's rows before the
      // reverse pass was measured and is no faster: 0.1037 against 0.1019 ms at chunk 128).
      constexpr int SEG = KT >= 3 ? 2 : 4;
      const unsigned xp = opaque(xpitch);
      float dots[RPL];  // the rows' dots, summed over the wave (the same in every lane)
      const unsigned me = (unsigned)lane_now();
      // r: a[i+1] * d[i+1] on entry for the wave's last row (what the rows after the group hand in),
      // d[i+1] itself for the others, where d[i] = dy[i] + a[i+1] * d[i+1] is one multiply-add
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = sR[grp][me * CPL + e];
#pragma unroll
      for (int i0 = RPL - SEG; i0 >= 0; i0 -= SEG) {
        __builtin_amdgcn_sched_barrier(0);
        float ym[CPL];  // forward value of the row before the segment
#pragma unroll
        for (int e = 0; e < CPL; ++e) ym[e] = sS[t][grp][me * CPL + e];
#pragma unroll
        for (int i = 0; i < i0; ++i)
#pragma unroll
          for (int e = 0; e < CPL; ++e) ym[e] = fmaf(a[i], ym[e], row_get<T, NW>(xr[t][i], e));
        float yv[SEG - 1][CPL];  // forward values of the segment's rows but the last
        {
          float s[CPL];
#pragma unroll
          for (int e = 0; e < CPL; ++e) s[e] = ym[e];
#pragma unroll
          for (int i = 0; i < SEG - 1; ++i)
#pragma unroll
            for (int e = 0; e < CPL; ++e) {
              s[e] = fmaf(a[i0 + i], s[e], row_get<T, NW>(xr[t][i0 + i], e));
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
            const float d = i == RPL - 1 ? row_get<T, NW>(dr[i], e) + r[e] : fmaf(a[i + 1 < RPL ? i + 1 : i], r[e], row_get<T, NW>(dr[i], e));
            dot = fmaf(d, j > 0 ? yv[j - 1][e] : ym[e], dot);
            r[e] = d;
          }
          if (more) xr[t][i] = flat_load_row<NW>(xdn, col_off(nx, (int)me) + row_off(t, i, xp));
          dots[i] = wave_sum(dot) * a[i];
        }
      }
      {
        // (rows at or past the limit have dy = 0 and give 0); a scalar base and the lane's row as a
        // 32-bit offset, formed here and not kept
        float total = 0.f;  // lane i reports row i of the wave
#pragma unroll
        for (int i = 0; i < RPL; ++i)
          if (me == (unsigned)i) total = dots[i];
        const int row = (int)me;
        const int q0 = kTileRows * t + RPL * grp;
        float* pb = part + ((it.chunk_id * ntiles + it.ctile) * (int64_t)Q + q0);
        if (me < (unsigned)RPL && q0 + row < Q) pb[row] = total;
      }
    }
    if (more) {
      araw = coef_load(nx);
    }
    w = wn;
    it = nx;
  }
}

// ------------------------------------------------------------------------------------
// The same for chunks of more than four sub-tiles (up to EMA_MAX_CHUNK rows), whose x rows do not fit
// the registers: x is read twice.  A first walk over the sub-tiles 0 .. K-2 only finds the forward
// state at every sub-tile boundary (local pass, one chain over the row groups, nothing kept but BN
// floats per boundary); the second walk, from the last sub-tile to the first, reads x again next to
// dy and does what da_flat_kernel does per sub-tile, with the local forward pass and the forward
// chain inside the step.  The decays of the whole chunk sit in LDS (one thread per row forms them
// at the start of a chunk).  Traffic: (3 K - 1) / (2 K) of the algorithmic bytes' x + dy.
// ------------------------------------------------------------------------------------
template <typename T, int CPL, int RPL>
struct FlatLongCfg {
  using W = TileCfg<T, CPL, RPL>;
  static constexpr int kMaxSub = EMA_MAX_CHUNK_DEV / kTileRows;
  static constexpr int kFloats = 2 * W::NG * W::BN    // forward and reverse group states
                                 + kMaxSub * W::BN    // forward state at the sub-tile boundaries
                                 + EMA_MAX_CHUNK_DEV  // the chunk's decays
                                 + W::NG + 4;         // group decays, flag
  static constexpr int kRowBytes = W::BN * (int)sizeof(T);
  static constexpr int smem_bytes = kFloats * (int)sizeof(float) + kTileRows * kRowBytes;
  static_assert(kFloats % 4 == 0, "the staged rows start at a multiple of 16 bytes");
  static_assert(smem_bytes <= 160 * 1024, "LDS of one compute unit");
};

template <typename T, int CPL, int RPL>
__global__ __launch_bounds__(64 * (kTileRows / RPL), 1) void da_flat_long_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ cs, float* __restrict__ part, int* __restrict__ steep, int nh, int L, int Tdim,
    int Q, int C, int ntiles, int total) {
  using W = TileCfg<T, CPL, RPL>;
  using F = FlatLongCfg<T, CPL, RPL>;
  constexpr int BN = W::BN, NW = W::NW, NG = W::NG, NT = W::NT;
  static_assert(2 * BN <= NT, "one thread per column and direction");
  static_assert(NT >= EMA_MAX_CHUNK_DEV, "one thread per row of a chunk");
  extern __shared__ __attribute__((aligned(16))) float flat_smem[];
  float (*sS)[BN] = reinterpret_cast<float (*)[BN]>(flat_smem);
  float (*sR)[BN] = reinterpret_cast<float (*)[BN]>(flat_smem + NG * BN);
  float (*sY)[BN] = reinterpret_cast<float (*)[BN]>(flat_smem + 2 * NG * BN);
  float* const sA = flat_smem + 2 * NG * BN + F::kMaxSub * BN;
  float* const sD = sA + EMA_MAX_CHUNK_DEV;
  int* const sFlag = reinterpret_cast<int*>(sD + NG);
  const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  constexpr int ROWB = F::kRowBytes, LPR = ROWB / 16, RPI = 64 / LPR, NCOPY = RPL / RPI;
  static_assert(RPL % RPI == 0, "whole rows per copy");
  char* const stage = reinterpret_cast<char*>(flat_smem + F::kFloats) + grp * (RPL * ROWB);
  const int K = (Q + kTileRows - 1) / kTileRows;

  auto opaque = [](unsigned v) {
    asm volatile("" : "+s"(v));
    return v;
  };
  if (threadIdx.x == 0) *sFlag = 0;
  __syncthreads();
  auto lane_now = [&]() {
    return (int)__builtin_amdgcn_mbcnt_hi(opaque(~0u), __builtin_amdgcn_mbcnt_lo(opaque(~0u), 0u));
  };
  struct Item {
    int64_t chunk_id, xbase, dbase;
    int ctile, limit, ncols;
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
    it.xbase = b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl + col0;
    it.dbase = b * sd.sb + h * sd.sh + (int64_t)c * Q * sd.sl + col0;
    return it;
  };
  const unsigned xpitch = (unsigned)sx.sl * (unsigned)sizeof(T), dpitch = (unsigned)sd.sl * (unsigned)sizeof(T);
  // the x rows of this wave in sub-tile t of chunk c, through the chunk's descriptor
  auto x_request = [&](RowWords<NW>* rows, __amdgpu_buffer_rsrc_t desc, const Item& c, int t) {
    const int ln = lane_now();
    const unsigned col = ln * CPL < c.ncols ? (unsigned)ln * (unsigned)(CPL * sizeof(T)) : kFlatNoColumn;
    const unsigned row0 = (unsigned)(kTileRows * t + RPL * grp) * opaque(xpitch);
#pragma unroll
    for (int i = 0; i < RPL; ++i) rows[i] = flat_load_row<NW>(desc, col + row0 + (unsigned)i * xpitch);
  };
  // this thread's row of the chunk: cs[q] - cs[q-1] (cs[0] itself for row 0, 0 at or past the limit)
  auto coef_load = [&](const Item& c) {
    const int q = 64 * grp + lane_now();
    float raw = 0.f;
    if (q < c.limit) {
      const float* p = cs + c.chunk_id * Q + q;
      raw = p[0] - (q > 0 ? p[-1] : 0.f);
    }
    return raw;
  };
  auto dy_request = [&](const Item& c, int t) {
    const T* base = dy + c.dbase;
    const int me = lane_now();
    const unsigned colb = min((unsigned)(me % LPR) * 16u, (unsigned)c.ncols * (unsigned)sizeof(T) - 16u);
#pragma unroll
    for (int j = 0; j < NCOPY; ++j) {
      const int row = min(kTileRows * t + RPL * grp + RPI * j + me / LPR, c.limit - 1);
      flat_copy16_to_lds(base, (unsigned)row * dpitch + colb, stage + j * 1024);
    }
  };
  auto dy_take = [&](RowWords<NW>* rows, const Item& c, int t) {
    const int nrows = c.limit - (kTileRows * t + RPL * grp);
    const int ln = lane_now();
    const bool cok = ln * CPL < c.ncols;
    const bool full = nrows >= RPL && __all(cok);
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      rows[i] = *reinterpret_cast<const RowWords<NW>*>(stage + i * ROWB + ln * (CPL * (int)sizeof(T)));
      if (!full && !(i < nrows && cok)) rows[i] = row_zero<NW>();
    }
  };
  // the decays of this wave's rows of sub-tile t, from LDS into scalar registers
  auto decays = [&](float* a, int t) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) a[i] = wave_uniform(sA[kTileRows * t + RPL * grp + i]);
  };
  // local forward pass over the rows of a sub-tile: the group's state and decay into LDS
  auto local_forward = [&](const RowWords<NW>* rows, const float* a) {
    float s[CPL], D = 1.f;
#pragma unroll
    for (int e = 0; e < CPL; ++e) s[e] = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      D *= a[i];
#pragma unroll
      for (int e = 0; e < CPL; ++e) s[e] = fmaf(a[i], s[e], row_get<T, NW>(rows[i], e));
    }
    const int ln = lane_now();
#pragma unroll
    for (int e = 0; e < CPL; ++e) sS[grp][ln * CPL + e] = s[e];
    if (ln == 0) sD[grp] = D;
  };
  constexpr int CW = BN / 64;  // waves with one thread per column

  RowWords<NW> xr[RPL], dr[RPL];
  float craw = 0.f;
  int w = blockIdx.x;
  Item it = decode(w < total ? w : 0);
  if (w < total) {
    x_request(xr, flat_rows_desc(x + it.xbase, sx.sl, it.limit, it.ncols), it, 0);
    craw = coef_load(it);
  }
  while (w < total) {
    const int wn = w + (int)gridDim.x;
    const bool more = wn < total;
    const Item nx = decode(more ? wn : 0);
    const __amdgpu_buffer_rsrc_t xd = flat_rows_desc(x + it.xbase, sx.sl, it.limit, it.ncols);
    const __amdgpu_buffer_rsrc_t xdn = flat_rows_desc(x + nx.xbase, sx.sl, nx.limit, nx.ncols);
    {
      // the chunk's decays, the flag of a rising cumsum, a zero state before the first row
      const int ln = lane_now(), q = 64 * grp + ln;
      sA[q] = __expf(fminf(craw, 0.f));
      if (__any(craw > 0.f && q > 0) && ln == 0) *sFlag = 1;
      if (q < BN) sY[0][q] = 0.f;
    }
    __syncthreads();

    // 1. the forward state at the sub-tile boundaries
    for (int t = 0; t < K - 1; ++t) {
      float a[RPL];
      decays(a, t);
      local_forward(xr, a);
      rows_opaque<NW, RPL>(xr);
      // the rows of the sub-tile after this one, which the next step needs whichever walk it belongs
      // to; before the last of them the copies of the last sub-tile's dy rows
      if (t == K - 2) dy_request(it, K - 1);
      x_request(xr, xd, it, t + 1);
      __syncthreads();
      if (grp < CW) {
        const int k = 64 * grp + lane_now();
        float sg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) sg[g] = sS[g][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[g]);
        float E = sY[t][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) E = fmaf(dg[g], E, sg[g]);
        sY[t + 1][k] = E;
      }
      __syncthreads();
    }

    // 2. sub-tiles from the last to the first
    float h_in = 0.f;  // chain threads: reverse state entering the sub-tile from the rows after it
    for (int t = K - 1; t >= 0; --t) {
      // The copies of this sub-tile's dy rows were requested a step ago and the RPL x rows of this step
      // after them: once at most RPL newer operations are under way they have landed.
      __builtin_amdgcn_sched_barrier(0);
      flat_wait_loads<RPL>();
      dy_take(dr, it, t);
      if (t > 0) dy_request(it, t - 1);
      __builtin_amdgcn_sched_barrier(0);
      float a[RPL];
      decays(a, t);
      // 2a. local passes: reverse over dy (u[i] = dy[i] + a[i+1] * u[i+1]; the group hands on a[0] * u[0]),
      // forward over x
      float r[CPL];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = row_get<T, NW>(dr[RPL - 1], e);
#pragma unroll
      for (int i = RPL - 2; i >= 0; --i)
#pragma unroll
        for (int e = 0; e < CPL; ++e) r[e] = fmaf(a[i + 1], r[e], row_get<T, NW>(dr[i], e));
      {
        const int ln = lane_now();
#pragma unroll
        for (int e = 0; e < CPL; ++e) sR[grp][ln * CPL + e] = r[e] * a[0];
      }
      local_forward(xr, a);
      rows_opaque<NW, RPL>(dr);
      rows_opaque<NW, RPL>(xr);
      __syncthreads();

      // 2b. chains over the row groups
      if (grp < CW) {
        const int k = 64 * grp + lane_now();
        if (t == K - 1 && k == 0) {
          if (it.ctile == 0) steep[it.chunk_id] = *sFlag;
          *sFlag = 0;
        }
        float rg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) rg[g] = sR[g][k];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[g]);
#pragma unroll
        for (int g = NG - 1; g >= 0; --g) {
          sR[g][k] = h_in;
          h_in = fmaf(dg[g], h_in, rg[g]);
        }
      } else if (grp < 2 * CW) {
        const int kf = 64 * (grp - CW) + lane_now();
        float sg[NG], dg[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) sg[g] = sS[g][kf];
#pragma unroll
        for (int g = 0; g < NG; ++g) dg[g] = wave_uniform(sD[g]);
        float E = sY[t][kf];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          sS[g][kf] = E;
          E = fmaf(dg[g], E, sg[g]);
        }
      }
      __syncthreads();

      // 2c. reverse pass with the dots, in two segments of the wave's rows (as in da_flat_kernel);
      // behind the last use of an x row the same row of the step after this one is requested
      constexpr int SEG = 4;
      const unsigned me = (unsigned)lane_now();
      const bool next_x = t > 0 || more;
      const __amdgpu_buffer_rsrc_t xnext = t > 0 ? xd : xdn;
      const unsigned xcol = (t > 0 ? (int)me * CPL < it.ncols : (int)me * CPL < nx.ncols)
                                ? me * (unsigned)(CPL * sizeof(T)) : kFlatNoColumn;
      const unsigned xrow0 = (unsigned)(kTileRows * (t > 0 ? t - 1 : 0) + RPL * grp) * opaque(xpitch);
      float dots[RPL];
#pragma unroll
      for (int e = 0; e < CPL; ++e) r[e] = sR[grp][me * CPL + e];
#pragma unroll
      for (int i0 = RPL - SEG; i0 >= 0; i0 -= SEG) {
        __builtin_amdgcn_sched_barrier(0);
        float ym[CPL];
#pragma unroll
        for (int e = 0; e < CPL; ++e) ym[e] = sS[grp][me * CPL + e];
#pragma unroll
        for (int i = 0; i < i0; ++i)
#pragma unroll
          for (int e = 0; e < CPL; ++e) ym[e] = fmaf(a[i], ym[e], row_get<T, NW>(xr[i], e));
        float yv[SEG - 1][CPL];
        {
          float s[CPL];
#pragma unroll
          for (int e = 0; e < CPL; ++e) s[e] = ym[e];
#pragma unroll
          for (int i = 0; i < SEG - 1; ++i)
#pragma unroll
            for (int e = 0; e < CPL; ++e) {
              s[e] = fmaf(a[i0 + i], s[e], row_get<T, NW>(xr[i0 + i], e));
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
            const float d = i == RPL - 1 ? row_get<T, NW>(dr[i], e) + r[e] : fmaf(a[i + 1 < RPL ? i + 1 : i], r[e], row_get<T, NW>(dr[i], e));
            dot = fmaf(d, j > 0 ? yv[j - 1][e] : ym[e], dot);
            r[e] = d;
          }
          if (next_x) xr[i] = flat_load_row<NW>(xnext, xcol + xrow0 + (unsigned)i * xpitch);
          dots[i] = wave_sum(dot) * a[i];
        }
      }
      {
        float total = 0.f;  // lane i reports row i of the wave
#pragma unroll
        for (int i = 0; i < RPL; ++i)
          if (me == (unsigned)i) total = dots[i];
        const int q0 = kTileRows * t + RPL * grp;
        float* pb = part + ((it.chunk_id * ntiles + it.ctile) * (int64_t)Q + q0);
        if (me < (unsigned)RPL && q0 + (int)me < Q) pb[me] = total;
      }
    }
    if (more) craw = coef_load(nx);
    w = wn;
    it = nx;
  }
}

}  // namespace ema
