// HBM-bound kernels of the EMA chunked scan: cumsum, decay-weighted chunk reductions,
// inter-chunk recurrences (forward and reverse), row dots for the log-decay gradient and
// the final combination.  Device code only; launched from ema_abi.hip.
#pragma once
#include "ema_device.h"

namespace ema {

// ------------------------------------------------------------------------------------
// Measurement aid: the plainest streaming kernel, one 16-byte piece per thread, non-temporal;
// dst = a (one source) or dst = a ^ b (two sources).  What it sustains is the practical ceiling
// the scan kernels are held against.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                          uint4* __restrict__ dst, int64_t n16) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n16) return;
  u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a) + i);
  if (b) v ^= __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(b) + i);
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst) + i);
}

// ------------------------------------------------------------------------------------
// Copies in the access pattern of the single-pass kernels (measurement aids).  The tensor is
// (slabs, rows, row_bytes) bytes; a tile is 128 rows x 512 bytes; one persistent workgroup per
// compute unit takes the tiles in chunk-major order (all slabs and row pieces of rows 0..127, then
// of rows 128..255, ...), workgroup w the tiles w, w + grid, ...; a lane moves 8 bytes of each of
// its rows, a wave's loads of a tile all go out before its stores.
//   tile_copy_shape_kernel<16>: sixteen waves, wave g moves rows 8 g .. 8 g + 7: the shape in which
//             fwd_tile_kernel and bwd_tile_kernel load and store;
//   tile_copy_shape_kernel<8>:  eight waves with 16 consecutive rows each;
//   tile_copy_kernel:           eight waves, instruction i of wave g moves row (8 i + g + slab) % 128:
//             the rows of a wave are 8 apart, the waves of a workgroup touch neighbouring rows, and
//             slabs (whose addresses differ by a large power of two) are rotated against each other.
// At b16 nh2 d1024 L4096, bfloat16, these sustain 5.5, 5.4 and 6.0 TB/s; the first with two inputs 5.9 TB/s.
// ------------------------------------------------------------------------------------
// (src2, if not null: a second input of the same layout; dst = src ^ src2, as in the backward kernel's
// two inputs and one output)
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void tile_copy_shape_kernel(const char* __restrict__ src,
                                                                     const char* __restrict__ src2, char* __restrict__ dst,
                                                                     int slabs, int row_blocks, int pieces,
                                                                     int64_t row_bytes, int64_t slab_bytes) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  constexpr int RPW = 128 / WAVES;  // rows of a wave
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int per_block = slabs * pieces, total = row_blocks * per_block;
  for (int id = blockIdx.x; id < total; id += gridDim.x) {
    const int rb = id / per_block, r = id - rb * per_block;
    const int slab = r / pieces, piece = r - slab * pieces;
    const int64_t base = (int64_t)slab * slab_bytes + ((int64_t)rb * 128 + RPW * g) * row_bytes + (int64_t)piece * 512 + lane * 8;
    u32x2 v[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src + base + i * row_bytes));
    if (src2) {
      u32x2 u[RPW];
#pragma unroll
      for (int i = 0; i < RPW; ++i) u[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src2 + base + i * row_bytes));
#pragma unroll
      for (int i = 0; i < RPW; ++i) v[i] ^= u[i];
    }
#pragma unroll
    for (int i = 0; i < RPW; ++i) __builtin_nontemporal_store(v[i], reinterpret_cast<u32x2*>(dst + base + i * row_bytes));
  }
}

__global__ __launch_bounds__(512) void tile_copy_kernel(const char* __restrict__ src, char* __restrict__ dst,
                                                        int slabs, int row_blocks, int pieces, int64_t row_bytes,
                                                        int64_t slab_bytes) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int per_block = slabs * pieces, total = row_blocks * per_block;
  for (int id = blockIdx.x; id < total; id += gridDim.x) {
    const int rb = id / per_block, r = id - rb * per_block;
    const int slab = r / pieces, piece = r - slab * pieces;
    const int64_t base = (int64_t)slab * slab_bytes + (int64_t)rb * 128 * row_bytes + (int64_t)piece * 512 + lane * 8;
    u32x2 v[16];
    int row[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) row[i] = (8 * i + g + slab) & 127;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src + base + row[i] * row_bytes));
#pragma unroll
    for (int i = 0; i < 16; ++i) __builtin_nontemporal_store(v[i], reinterpret_cast<u32x2*>(dst + base + row[i] * row_bytes));
  }
}

// The same copy with the interleaved order on the memory side and consecutive rows per wave in
// registers, as a scanning kernel would need them: rows arrive interleaved, pass through a 64 KB
// tile in LDS to the wave that owns them, and go back through a second tile to be stored
// interleaved; the next tile's rows are requested while the current one is exchanged.
__global__ __launch_bounds__(512) void tile_copy_exchange_kernel(const char* __restrict__ src, char* __restrict__ dst,
                                                                 int slabs, int row_blocks, int pieces, int64_t row_bytes,
                                                                 int64_t slab_bytes) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x2* tin = reinterpret_cast<u32x2*>(smem);
  u32x2* tout = reinterpret_cast<u32x2*>(smem + 128 * 512);
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int per_block = slabs * pieces, total = row_blocks * per_block;
  auto base_of = [&](int id, int& slab) {
    const int rb = id / per_block, r = id - rb * per_block;
    slab = r / pieces;
    const int piece = r - slab * pieces;
    return (int64_t)slab * slab_bytes + (int64_t)rb * 128 * row_bytes + (int64_t)piece * 512 + lane * 8;
  };
  u32x2 v[16];
  int id = blockIdx.x, slab = 0;
  int64_t base = 0;
  if (id < total) {
    base = base_of(id, slab);
#pragma unroll
    for (int i = 0; i < 16; ++i)
      v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src + base + ((8 * i + g + slab) & 127) * row_bytes));
  }
  while (id < total) {
#pragma unroll
    for (int i = 0; i < 16; ++i) tin[((8 * i + g + slab) & 127) * 64 + lane] = v[i];
    __syncthreads();
    u32x2 w[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i] = tin[(16 * g + i) * 64 + lane];
    const int cur_slab = slab;
    const int64_t cur_base = base;
    id += gridDim.x;
    if (id < total) {
      base = base_of(id, slab);
#pragma unroll
      for (int i = 0; i < 16; ++i)
        v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src + base + ((8 * i + g + slab) & 127) * row_bytes));
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) tout[(16 * g + i) * 64 + lane] = w[i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = (8 * i + g + cur_slab) & 127;
      __builtin_nontemporal_store(tout[row * 64 + lane], reinterpret_cast<u32x2*>(dst + cur_base + row * row_bytes));
    }
  }
}

// ------------------------------------------------------------------------------------
// F1: per-chunk inclusive cumsum of the log-decay.  One wave per (n, c); lane l owns the
// `per` consecutive positions starting at l * per, sums them serially, and the lane totals
// are scanned across the wave with DPP.  With prob != 0 the input holds probabilities p and
// the log-decay is log(1 - p).
// ------------------------------------------------------------------------------------
// A probability with its sign bit set marks the first position of a packed sequence: nothing
// survives it, a log-decay of -inf.
__device__ __forceinline__ float cumsum_term(float v, int prob) {
  if (!prob) return v;
  return (__float_as_uint(v) >> 31) ? -INFINITY : log1pf(-v);
}

// The work of workgroup `block` (four chunks, one per wave).
__device__ __forceinline__ void cumsum_block(int64_t block, const float* __restrict__ A, SeqStrides sa,
                                             float* __restrict__ cs, int nh, int L, int Q, int C,
                                             int64_t total_chunks, int prob) {
  const int lane = threadIdx.x & 63;
  const int64_t chunk_id = block * 4 + (threadIdx.x >> 6);
  if (chunk_id >= total_chunks) return;
  const int64_t n = chunk_id / C;
  const int c = (int)(chunk_id - n * C);
  const int64_t b = n / nh;
  const int h = (int)(n - b * nh);
  const int per = (Q + 63) >> 6;
  const int q0 = lane * per;
  const int limit = min(Q, L - c * Q);
  const float* a = A + b * sa.sb + h * sa.sh + (int64_t)c * Q * sa.sl;

  float local = 0.f;
  for (int i = 0; i < per; ++i) {
    const int q = q0 + i;
    if (q < limit) local += cumsum_term(a[(int64_t)q * sa.sl], prob);
  }
  float run = wave_exclusive_scan(local);  // prefix of the lane totals before this lane
  float* out = cs + chunk_id * Q;
  for (int i = 0; i < per; ++i) {
    const int q = q0 + i;
    if (q < limit) run += cumsum_term(a[(int64_t)q * sa.sl], prob);
    if (q < Q) out[q] = run;
  }
}

__global__ __launch_bounds__(256) void cumsum_kernel(const float* __restrict__ A,
                                                     SeqStrides sa, float* __restrict__ cs,
                                                     int nh, int L, int Q, int C,
                                                     int64_t total_chunks, int prob) {
  cumsum_block(blockIdx.x, A, sa, cs, nh, L, Q, C, total_chunks, prob);
}

// ------------------------------------------------------------------------------------
// F2 / B1: out[n,c,t] = sum_q w[q] * x[n, cQ+q, t] with
//   MODE 0 (chunk state):  w[q] = exp(min(cs[Q-1] - cs[q], 0))
//   MODE 1 (dstates):      w[q] = exp(cs[q])
// One workgroup per (n, c, column tile).  Threads are laid out as cg column groups (one
// 16-byte vector each) by 256/cg row lanes; every row lane strides over the chunk's rows
// with 16-byte coalesced loads, and the row lanes are then summed through LDS.
// ------------------------------------------------------------------------------------
template <typename T, int MODE>
__global__ __launch_bounds__(256) void chunk_reduce_kernel(
    const T* __restrict__ x, SeqStrides sx, const float* __restrict__ cs,
    float* __restrict__ out, int nh, int L, int Tdim, int Q, int C, int cg_log2, int ntiles) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float red[256 * VEC];
  const int tid = threadIdx.x;
  const int cg = 1 << cg_log2;
  const int col_group = tid & (cg - 1);
  const int row_lane = tid >> cg_log2;
  const int rows_par = 256 >> cg_log2;

  const int64_t blk = blockIdx.x;
  const int tile = (int)(blk % ntiles);
  const int64_t chunk_id = blk / ntiles;
  const int64_t n = chunk_id / C;
  const int c = (int)(chunk_id - n * C);
  const int64_t b = n / nh;
  const int h = (int)(n - b * nh);
  const int limit = min(Q, L - c * Q);
  const int col = (tile * cg + col_group) * VEC;
  const bool col_ok = col < Tdim;

  const float* csp = cs + chunk_id * Q;
  const float cs_last = csp[Q - 1];
  const T* xp = x + b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl + col;

  float acc[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = 0.f;

  constexpr int U = 4;
  const T* xq = col_ok ? xp : xp - col;  // a column tile past the end reads column 0 and is discarded
  for (int q0 = row_lane; q0 < limit; q0 += rows_par * U) {
    Vec16<T> v[U];
    float w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // unconditional loads from an index clamped into the chunk (a load inside a branch has to
      // complete before the next one is issued); what lies outside gets weight 0
      const int q = q0 + u * rows_par;
      const int qc = min(q, limit - 1);
      v[u] = load16_stream(xq + (int64_t)qc * sx.sl);
      const float a = csp[qc];
      const float wt = MODE == 0 ? __expf(fminf(cs_last - a, 0.f)) : __expf(a);
      w[u] = (q < limit && col_ok) ? wt : 0.f;
      if (!(q < limit && col_ok)) v[u].zero();
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] = fmaf(w[u], v[u].get(i), acc[i]);
  }

  // red[row_lane][col_group][i]
#pragma unroll
  for (int i = 0; i < VEC; ++i) red[(row_lane * cg + col_group) * VEC + i] = acc[i];
  __syncthreads();
  // thread tid sums column (tid) of the tile over the row lanes, then a second pass for
  // the remaining columns (cg * VEC may exceed 256).
  for (int j = tid; j < cg * VEC; j += 256) {
    float s = 0.f;
    for (int r = 0; r < rows_par; ++r) s += red[r * cg * VEC + j];
    const int ocol = tile * cg * VEC + j;
    if (ocol < Tdim) out[chunk_id * Tdim + ocol] = s;
  }
}

// ------------------------------------------------------------------------------------
// F3: forward inter-chunk recurrence.  One thread per (n, t); the running state stays in
// a register, chunk-local states are fetched U chunks ahead of the dependent FMAs.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void state_passing_fwd_kernel(
    const float* __restrict__ states, const float* __restrict__ cs_last, int64_t cl_sn,
    int64_t cl_sc, float* __restrict__ prev, float* __restrict__ final_state, int C,
    int Tdim, int tiles_per_seq) {
  const int64_t n = blockIdx.x / tiles_per_seq;
  const int t = (int)(blockIdx.x % tiles_per_seq) * 256 + threadIdx.x;
  if (t >= Tdim) return;
  const float* st = states + n * (int64_t)C * Tdim + t;
  float* pv = prev + n * (int64_t)C * Tdim + t;
  const float* cl = cs_last + n * cl_sn;
  float S = 0.f;
  constexpr int U = 8;
  for (int c0 = 0; c0 < C; c0 += U) {
    float s[U], a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;
      s[u] = c < C ? st[(int64_t)c * Tdim] : 0.f;
      a[u] = c < C ? cl[(int64_t)c * cl_sc] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;
      if (c < C) {
        pv[(int64_t)c * Tdim] = S;
        S = fmaf(__expf(a[u]), S, s[u]);
      }
    }
  }
  final_state[n * Tdim + t] = S;
}

// ------------------------------------------------------------------------------------
// B2: reverse inter-chunk recurrence.  One thread per (n, t).  With DOTS, besides g, every
// wave writes its partial of <prev[n,c], g[n,c]> to part[(n*C + c) * nw + wave_of_t]; the
// partials are summed (and scaled by exp(cs_last)) by state_passing_bwd_finish_kernel.
// ------------------------------------------------------------------------------------
template <bool DOTS>
__global__ __launch_bounds__(256) void state_passing_bwd_kernel(
    const float* __restrict__ prev, const float* __restrict__ cs_last, int64_t cl_sn,
    int64_t cl_sc, const float* __restrict__ ds, float* __restrict__ g,
    float* __restrict__ part, int C, int Tdim, int tiles_per_seq, int nw) {
  const int64_t n = blockIdx.x / tiles_per_seq;
  const int tile = (int)(blockIdx.x % tiles_per_seq);
  const int t = tile * 256 + threadIdx.x;
  const bool ok = t < Tdim;
  const int wave_id = tile * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t base = n * (int64_t)C * Tdim + (ok ? t : 0);
  const float* cl = cs_last + n * cl_sn;
  float cur = 0.f;
  constexpr int U = 8;
  for (int c1 = C - 1; c1 >= 0; c1 -= U) {
    float d[U], p[U], a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c1 - u;
      const bool in = c >= 0;
      d[u] = (in && ok) ? ds[base + (int64_t)c * Tdim] : 0.f;
      p[u] = (DOTS && in && ok) ? prev[base + (int64_t)c * Tdim] : 0.f;
      a[u] = in ? cl[(int64_t)c * cl_sc] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c1 - u;
      if (c >= 0) {  // uniform across the wave
        if (ok) g[base + (int64_t)c * Tdim] = cur;
        if (DOTS) {
          const float dot = wave_sum(p[u] * cur);
          if (lane == 0 && wave_id < nw) part[(n * C + c) * (int64_t)nw + wave_id] = dot;
        }
        cur = fmaf(__expf(a[u]), cur, d[u]);
      }
    }
  }
}

__global__ __launch_bounds__(256) void state_passing_bwd_finish_kernel(
    const float* __restrict__ part, const float* __restrict__ cs_last, int64_t cl_sn,
    int64_t cl_sc, float* __restrict__ ddA_chunk, int C, int nw, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t n = i / C;
  const int c = (int)(i - n * C);
  float s = 0.f;
  for (int w = 0; w < nw; ++w) s += part[i * nw + w];
  ddA_chunk[i] = c == 0 ? 0.f : __expf(cs_last[n * cl_sn + (int64_t)c * cl_sc]) * s;
}

// ------------------------------------------------------------------------------------
// B4 / B5: per-row dot products against a per-chunk vector.
//   MODE 0 (db): r[m] = exp(min(cs[Q-1]-cs[m],0)) * <g[n,c], x[n,cQ+m]>, rows past the
//                chunk limit give 0; out[0] = 0, out[j] = r[j-1] (raw) or
//                out[j] = sum_{m<j} r[m] (cumulative).
//   MODE 1 (dc): out[m] = exp(cs[m]) * <dy[n,cQ+m], prev[n,c]>, 0 past the limit.
// One workgroup of kRowDotThreads per (n, c); wave w takes rows R*w + R*NWV*i + {0..R-1}; a wave
// covers the feature axis with 16-byte loads per lane (R of them in flight per lane and column
// step) and reduces with DPP.
// ------------------------------------------------------------------------------------
constexpr int kRowDotThreads = 512;
template <typename T, int MODE>
__global__ __launch_bounds__(kRowDotThreads) void row_dot_kernel(const T* __restrict__ x, SeqStrides sx,
                                                                 const float* __restrict__ vec,
                                                                 const float* __restrict__ cs,
                                                                 float* __restrict__ out, int nh, int L,
                                                                 int Tdim, int Q, int C, int raw) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int NWV = kRowDotThreads / 64;
  __shared__ float rbuf[EMA_MAX_CHUNK_DEV];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int64_t chunk_id = blockIdx.x;
  const int64_t n = chunk_id / C;
  const int c = (int)(chunk_id - n * C);
  const int64_t b = n / nh;
  const int h = (int)(n - b * nh);
  const int limit = min(Q, L - c * Q);
  const float* csp = cs + chunk_id * Q;
  const float cs_last = csp[Q - 1];
  const float* vp = vec + chunk_id * Tdim;
  const T* xp = x + b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl;

  // rows per wave and turn.  Measured at b16 nh2 d1024 L4096 chunk 128 (db / dc, us): 8 rows 50 / 49, 4 rows
  // 47.5 / 47, 2 rows 44.7 / 44.5, 1 row 47.7 / 47.5, 16 rows 58 / 56: fewer registers per wave keep more waves
  // resident, and two 16-byte loads per lane and column step are enough to cover the latency with them.
  constexpr int R = 2;
  for (int m0 = wave * R; m0 < Q; m0 += NWV * R) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    for (int col = lane * VEC; col < Tdim; col += 64 * VEC) {
      float gv[VEC];
#pragma unroll
      for (int i = 0; i < VEC; i += 4) {
        const float4 t4 = *reinterpret_cast<const float4*>(vp + col + i);
        gv[i] = t4.x; gv[i + 1] = t4.y; gv[i + 2] = t4.z; gv[i + 3] = t4.w;
      }
      Vec16<T> v[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        v[r] = load16_stream(xp + (int64_t)min(m0 + r, limit - 1) * sx.sl + col);
        if (m0 + r >= limit) v[r].zero();
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[r] = fmaf(gv[i], v[r].get(i), acc[r]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float s = wave_sum(acc[r]);
      const int m = m0 + r;
      if (lane == 0 && m < Q) {
        float w = 0.f;
        if (m < limit) w = MODE == 0 ? __expf(fminf(cs_last - csp[m], 0.f)) : __expf(csp[m]);
        rbuf[m] = w * s;
      }
    }
  }
  __syncthreads();
  float* op = out + chunk_id * Q;
  if (MODE == 1) {
    for (int m = tid; m < Q; m += kRowDotThreads) op[m] = rbuf[m];
  } else if (raw) {
    for (int m = tid; m < Q; m += kRowDotThreads) op[m] = m == 0 ? 0.f : rbuf[m - 1];
  } else if (wave == 0) {
    // out[j] = sum_{m<j} r[m]: exclusive scan, lane l owns positions l*per .. l*per+per-1
    const int per = (Q + 63) >> 6;
    const int q0 = lane * per;
    float local = 0.f;
    for (int i = 0; i < per; ++i)
      if (q0 + i < Q) local += rbuf[q0 + i];
    float run = wave_exclusive_scan(local);
    for (int i = 0; i < per; ++i) {
      const int q = q0 + i;
      if (q < Q) {
        op[q] = run;
        run += rbuf[q];
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// Final sum of the log-decay gradient, one wave per (n, c):
//   ddA[j] = intra[j] + next[j] + sum_{m>=j} (s[m] + [m == Q-1] * ddA_chunk)
// (the reverse cumsum and the three-way add of the reference's combined backward).
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void combine_dA_kernel(const float* __restrict__ intra,
                                                         const float* __restrict__ next,
                                                         const float* __restrict__ sraw,
                                                         const float* __restrict__ ddA_chunk,
                                                         float* __restrict__ ddA, int Q,
                                                         int64_t total_chunks) {
  const int lane = threadIdx.x & 63;
  const int64_t chunk_id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk_id >= total_chunks) return;
  // Lane l owns the positions Q-1-p for p = l*per .. l*per+per-1, so a forward scan over
  // the lanes accumulates from the end of the chunk.
  const int per = (Q + 63) >> 6;
  const int p0 = lane * per;
  const float* sp = sraw + chunk_id * Q;
  const float extra = ddA_chunk[chunk_id];
  float local = 0.f;
  for (int i = 0; i < per; ++i) {
    const int p = p0 + i;
    if (p < Q) local += sp[Q - 1 - p] + (p == 0 ? extra : 0.f);
  }
  float run = wave_exclusive_scan(local);
  for (int i = 0; i < per; ++i) {
    const int p = p0 + i;
    if (p < Q) {
      const int q = Q - 1 - p;
      run += sp[q] + (p == 0 ? extra : 0.f);
      const int64_t o = chunk_id * Q + q;
      ddA[o] = intra[o] + next[o] + run;
    }
  }
}

}  // namespace ema
