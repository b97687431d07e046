// Intra-chunk kernels built on the block structure of the segsum-decay matrix.
//
// Inside a chunk the decay matrix M[m,k] = exp(cs[m] - cs[k]) (k <= m) is cut into 32-row
// blocks.  A diagonal 32 x 32 block is dense and goes through the MFMA; a block below the
// diagonal is the outer product exp(cs[m] - cs[e]) * exp(cs[e] - cs[k]) for any row e
// between the two blocks, so all of them together are applied as one rank-1 update per
// row block: a running state P_j (the scan value at the last row before block j), carried
// from block to block in f32.  The reverse (gradient) direction is the mirror image with
// a running state H_j referenced to the last row of block j.
//
// A workgroup of 4 waves owns a tile of 128 rows x BN columns; wave w owns block w:
//   1. the tile is staged in LDS with 16-byte coalesced loads;
//   2. wave w reduces its 32 rows to the block-local state s_w (f32 VALU);
//   3. the carried states P_0..P_4 are chained (one thread per column);
//   4. wave w multiplies its rows with the diagonal block on the MFMA (operands: the tile
//      through transposing LDS reads, the decay block built in registers as bf16 hi + lo),
//      starting the accumulators from exp(cs[m] - cs[e_{w-1}]) * P_w;
//   5. results are packed in LDS (over the wave's own input rows) and leave with 16-byte
//      coalesced stores.
#pragma once
#include "ema_device.h"

namespace ema {

constexpr int kTileRows = 128;

template <typename T, int BN>
struct WalkCfg {
  static constexpr int EPL = Vec16<T>::N;        // operand elements per lane and MFMA group
  static constexpr int KG = 2 * EPL;             // k extent of an MFMA group
  static constexpr int NG = 32 / KG;             // MFMA groups per 32-row block
  static constexpr int NDB = BN / 32;            // 32-column blocks per tile
  static constexpr int CPL = BN / 64;            // columns per lane in the block-state step
  static constexpr int ROW = BN + EPL;           // LDS pitch in elements (16 bytes of padding)
  static constexpr int TILE = kTileRows * ROW;   // elements of one staged tile
  static constexpr int VPR = BN / EPL;           // 16-byte vectors per row
  static constexpr int RPP = 256 / VPR;          // rows staged per pass of the workgroup
  static constexpr int TILE_BYTES = TILE * (int)sizeof(T);
  // f32 scratch after the tiles.  Kernels that scan in both directions (DIRS = 2) keep
  // csT[132] wf[128] wr[128] sj[4*BN] rj[4*BN] Pj[5*BN] Hj[5*BN]; one-directional kernels
  // (DIRS = 1) keep csT[132] w[128] s[4*BN] P[5*BN] and the two names of each pair alias.
  static constexpr int scratch_floats(int dirs) { return 132 + dirs * (128 + 4 * BN + 5 * BN); }
  static constexpr int smem_bytes(int ntiles, int dirs) {
    return ntiles * TILE_BYTES + scratch_floats(dirs) * (int)sizeof(float);
  }
};

struct WalkScratch {
  float *csT, *wf, *wr, *sj, *rj, *Pj, *Hj;
};

template <typename T, int BN, int DIRS>
__device__ __forceinline__ WalkScratch walk_scratch(unsigned char* smem, int ntiles) {
  float* f = reinterpret_cast<float*>(smem + ntiles * WalkCfg<T, BN>::TILE_BYTES);
  WalkScratch s;
  s.csT = f;
  s.wf = f + 132;
  s.wr = DIRS == 2 ? s.wf + 128 : s.wf;
  s.sj = s.wr + 128;
  s.rj = DIRS == 2 ? s.sj + 4 * BN : s.sj;
  s.Pj = s.rj + 4 * BN;
  s.Hj = DIRS == 2 ? s.Pj + 5 * BN : s.Pj;
  return s;
}

// Rows [tb, tb+128) x columns [col0, col0+BN) of one chunk into LDS; rows at or past
// `limit` and columns at or past Tdim are zero.  g points at (row 0 of the chunk, col 0).
template <typename T, int BN>
__device__ __forceinline__ void walk_load_tile(T* tile, const T* __restrict__ g, int64_t sl,
                                               int tb, int limit, int col0, int Tdim, int tid) {
  using C = WalkCfg<T, BN>;
  const int vcol = (tid % C::VPR) * C::EPL;
  const bool cok = col0 + vcol < Tdim;
  Vec16<T> v[kTileRows / C::RPP];
#pragma unroll
  for (int p = 0; p < kTileRows / C::RPP; ++p) {
    const int r = tid / C::VPR + p * C::RPP;
    // unconditional load from a row and column clamped into the tensor, zeroed afterwards
    v[p] = load16_stream(g + (int64_t)min(tb + r, limit - 1) * sl + (cok ? col0 + vcol : 0));
    if (tb + r >= limit || !cok) v[p].zero();
  }
#pragma unroll
  for (int p = 0; p < kTileRows / C::RPP; ++p) {
    const int r = tid / C::VPR + p * C::RPP;
    store16(&tile[r * C::ROW + vcol], v[p]);
  }
}

// csT[i] = cs[tb + i - 1] for i = 0..128 with cs[-1] := 0 and cs[q >= Q] := cs[Q-1];
// wf[t] = exp(cs[e_j] - cs[t]), wr[t] = exp(cs[t] - cs[e_{j-1}]) for row t of block j = t/32
// (e_j = last row of block j).  Thread t < 128 reads what it needs straight from global
// memory so that no barrier is needed between this and the tile load.
template <bool FWD, bool REV>
__device__ __forceinline__ void walk_load_cs(const WalkScratch& s, const float* __restrict__ csp,
                                             int tb, int Q, int tid) {
  auto at = [&](int q) { return q < 0 ? 0.f : csp[min(q, Q - 1)]; };
  if (tid < kTileRows) {
    const int j = tid >> 5;
    const float c_t = at(tb + tid);
    s.csT[tid + 1] = c_t;
    if (tid == 0) s.csT[0] = at(tb - 1);
    if (FWD) s.wf[tid] = __expf(fminf(at(tb + 32 * j + 31) - c_t, 0.f));
    if (REV) s.wr[tid] = __expf(fminf(c_t - at(tb + 32 * j - 1), 0.f));
  }
}

// out[w*BN + col] = sum_{k in block w} wts[32w + k] * tile[32w + k][col]; one wave per block,
// CPL adjacent columns per lane.
template <typename T, int BN>
__device__ __forceinline__ void walk_block_state(const T* tile, const float* wts, float* out,
                                                 int wave, int lane) {
  using C = WalkCfg<T, BN>;
  float s[C::CPL];
#pragma unroll
  for (int i = 0; i < C::CPL; ++i) s[i] = 0.f;
  const T* base = tile + (wave * 32) * C::ROW + C::CPL * lane;
#pragma unroll 8
  for (int k = 0; k < 32; ++k) {
    const float wt = wts[wave * 32 + k];
#pragma unroll
    for (int i = 0; i < C::CPL; ++i) s[i] = fmaf(wt, (float)base[k * C::ROW + i], s[i]);
  }
#pragma unroll
  for (int i = 0; i < C::CPL; ++i) out[wave * BN + C::CPL * lane + i] = s[i];
}

// Decay between the reference rows of consecutive blocks: exp(cs[e_j] - cs[e_{j-1}]).
__device__ __forceinline__ float walk_block_decay(const float* csT, int j) {
  return __expf(fminf(csT[32 * j + 32] - csT[32 * j], 0.f));
}

// Forward chain, thread t < BN: P_0 = carry-in; P_{j+1} = decay_j * P_j + s_j.  Pj[j*BN+t]
// for j = 0..4 (P_4 is the carry into the next tile).
template <int BN>
__device__ __forceinline__ void walk_chain_fwd(const WalkScratch& s, float p_in, int t) {
  float P = p_in;
  s.Pj[t] = P;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    P = fmaf(walk_block_decay(s.csT, j), P, s.sj[j * BN + t]);
    s.Pj[(j + 1) * BN + t] = P;
  }
}

// Reverse chain: H_3 = carry-in (referenced to the tile's last row);
// H_{j-1} = r_j + decay_j * H_j.  Hj[j*BN+t] for j = 0..3; Hj[4*BN+t] = H_{-1}, the carry
// into the previous tile.
template <int BN>
__device__ __forceinline__ void walk_chain_rev(const WalkScratch& s, float h_in, int t) {
  float H = h_in;
#pragma unroll
  for (int j = 3; j >= 0; --j) {
    s.Hj[j * BN + t] = H;
    H = fmaf(walk_block_decay(s.csT, j), H, s.rj[j * BN + t]);
  }
  s.Hj[4 * BN + t] = H;
}

// The diagonal decay block of wave w in MFMA operand layout: lane l holds, for row
// m = 32w + l%32, the factors of k = 32w + g*KG + EPL*(l/32) + e.
//   forward: (k <= m) * exp(cs[m] - cs[k]);  reverse: (k >= m) * exp(cs[k] - cs[m]).
// bf16 operands are split as hi + lo so that the product with the exact bf16 inputs keeps
// f32-grade accuracy; for f32 operands lo is unused.
template <typename T, bool REV>
__device__ __forceinline__ void walk_decay_frags(const float* csT, int wave, int lane,
                                                 Vec16<T>* hi, Vec16<T>* lo) {
  constexpr int EPL = Vec16<T>::N;
  constexpr int KG = 2 * EPL;
  constexpr int NG = 32 / KG;
  const int rm = 32 * wave + (lane & 31);
  const float cm = csT[rm + 1];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int k = 32 * wave + g * KG + EPL * (lane >> 5) + e;
      const float ck = csT[k + 1];
      const bool keep = REV ? (k >= rm) : (k <= rm);
      // branch-free: a masked element gets exp(-huge) = 0
      const float val = __expf(keep ? fminf(REV ? ck - cm : cm - ck, 0.f) : -1.0e30f);
      hi[g].set(e, val);
      if (sizeof(T) == 2) lo[g].set(e, val - hi[g].get(e));
    }
  }
}

// Input operand of one MFMA group: lane l gets tile[k0 + EPL*(l/32) + e][col0 + l%32].
__device__ __forceinline__ Vec16<bf16_t> walk_in_frag(const bf16_t* tile, int pitch, int k0,
                                                      int col0, int lane) {
  return lds_read_kmajor(tile, pitch, k0, col0, lane);
}
__device__ __forceinline__ Vec16<float> walk_in_frag(const float* tile, int pitch, int k0, int col0,
                                                     int lane) {
  Vec16<float> v;
  const float* p = tile + (k0 + 4 * (lane >> 5)) * pitch + col0 + (lane & 31);
  v.raw = make_float4(p[0], p[pitch], p[2 * pitch], p[3 * pitch]);
  return v;
}

// Transposed result block of wave w for the 32 columns starting at db*32: register v of
// lane l is out[row 32w + l%32][column db*32 + 8*(v/4) + 4*(l/32) + v%4].  Starts from
// u * carry[column] and adds the diagonal-block product.
template <typename T, int BN>
__device__ __forceinline__ floatx16 walk_block_mma(const T* tile, const Vec16<T>* hi,
                                                   const Vec16<T>* lo, const float* carry, float u,
                                                   int wave, int db, int lane) {
  using C = WalkCfg<T, BN>;
  floatx16 acc;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 p4 = *reinterpret_cast<const float4*>(&carry[db * 32 + 8 * q + 4 * (lane >> 5)]);
    acc[4 * q + 0] = u * p4.x;
    acc[4 * q + 1] = u * p4.y;
    acc[4 * q + 2] = u * p4.z;
    acc[4 * q + 3] = u * p4.w;
  }
#pragma unroll
  for (int g = 0; g < C::NG; ++g) {
    const Vec16<T> xf = walk_in_frag(tile, C::ROW, 32 * wave + g * C::KG, db * 32, lane);
    mma_group(xf, hi[g], acc);
    if (sizeof(T) == 2) mma_group(xf, lo[g], acc);
  }
  return acc;
}

// Packs a result block into the wave's own rows of an LDS tile (row-major, type T).
template <typename T, int BN>
__device__ __forceinline__ void walk_pack_block(T* tile, const floatx16& acc, int wave, int db,
                                                int lane) {
  using C = WalkCfg<T, BN>;
  T* rowp = tile + (32 * wave + (lane & 31)) * C::ROW + db * 32 + 4 * (lane >> 5);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if constexpr (sizeof(T) == 2) {
      typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
      bf16x4 pk;
      pk[0] = (bf16_t)acc[4 * q + 0];
      pk[1] = (bf16_t)acc[4 * q + 1];
      pk[2] = (bf16_t)acc[4 * q + 2];
      pk[3] = (bf16_t)acc[4 * q + 3];
      *reinterpret_cast<bf16x4*>(rowp + 8 * q) = pk;
    } else {
      *reinterpret_cast<float4*>(rowp + 8 * q) =
          make_float4(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
    }
  }
}

// The wave's 32 rows of an LDS tile to global memory, 16 bytes per lane.
template <typename T, int BN>
__device__ __forceinline__ void walk_store_rows(const T* tile, T* __restrict__ g, int64_t sl, int tb,
                                                int limit, int col0, int Tdim, int wave, int lane) {
  using C = WalkCfg<T, BN>;
  constexpr int RPW = 64 / C::VPR;  // rows per pass of one wave
  const int vcol = (lane % C::VPR) * C::EPL;
  if (col0 + vcol >= Tdim) return;
#pragma unroll
  for (int p = 0; p < 32 / RPW; ++p) {
    const int r = 32 * wave + p * RPW + lane / C::VPR;
    if (tb + r < limit)
      store16_stream(g + (int64_t)(tb + r) * sl + col0 + vcol, load16(&tile[r * C::ROW + vcol]));
  }
}

// ------------------------------------------------------------------------------------
// F4 (REV = false):
//   out[m,t] = exp(min(cs[m],0)) * vec[t] + sum_{k<=m} exp(min(cs[m]-cs[k],0)) * in[k,t]
// B3 (REV = true):
//   out[m,t] = exp(min(cs[Q-1]-cs[m],0)) * vec[t] + sum_{k>=m} exp(min(cs[k]-cs[m],0)) * in[k,t]
// for one chunk of any size Q: the workgroup walks the chunk's 128-row tiles in scan
// order, carrying the state across tiles in LDS.  Grid: (n, c, column tile).
// ------------------------------------------------------------------------------------
template <typename T, int BN, bool REV>
__global__ __launch_bounds__(256) void chunk_scan_walk_kernel(
    const T* __restrict__ in, SeqStrides si, const float* __restrict__ cs,
    const float* __restrict__ vec, T* __restrict__ out, SeqStrides so, int nh, int L, int Tdim,
    int Q, int C, int ntiles) {
  using Cfg = WalkCfg<T, BN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  const WalkScratch s = walk_scratch<T, BN, 1>(smem, 1);

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int ctile = (int)(blockIdx.x % ntiles);
  const int64_t chunk_id = blockIdx.x / ntiles;
  const int64_t n = chunk_id / C;
  const int c = (int)(chunk_id - n * C);
  const int64_t b = n / nh;
  const int h = (int)(n - b * nh);
  const int limit = min(Q, L - c * Q);
  const int col0 = ctile * BN;
  const float* csp = cs + chunk_id * Q;
  const T* ip = in + b * si.sb + h * si.sh + (int64_t)c * Q * si.sl;
  T* op = out + b * so.sb + h * so.sh + (int64_t)c * Q * so.sl;

  float carry = 0.f;  // thread t < BN: state of column col0 + t carried between tiles
  if (tid < BN && col0 + tid < Tdim) carry = vec[chunk_id * Tdim + col0 + tid];

  const int nrt = (Q + kTileRows - 1) / kTileRows;
  for (int it = 0; it < nrt; ++it) {
    const int tb = (REV ? nrt - 1 - it : it) * kTileRows;
    if (it) __syncthreads();
    walk_load_cs<!REV, REV>(s, csp, tb, Q, tid);
    walk_load_tile<T, BN>(tile, ip, si.sl, tb, limit, col0, Tdim, tid);
    __syncthreads();
    walk_block_state<T, BN>(tile, REV ? s.wr : s.wf, REV ? s.rj : s.sj, wave, lane);
    __syncthreads();
    if (tid < BN) {
      if (REV) {
        walk_chain_rev<BN>(s, carry, tid);
        carry = s.Hj[4 * BN + tid];
      } else {
        walk_chain_fwd<BN>(s, carry, tid);
        carry = s.Pj[4 * BN + tid];
      }
    }
    __syncthreads();
    Vec16<T> hi[Cfg::NG], lo[Cfg::NG];
    walk_decay_frags<T, REV>(s.csT, wave, lane, hi, lo);
    const float cm = s.csT[32 * wave + (lane & 31) + 1];
    const float u = REV ? __expf(fminf(s.csT[32 * wave + 32] - cm, 0.f))
                        : __expf(fminf(cm - s.csT[32 * wave], 0.f));
    const float* cr = (REV ? s.Hj : s.Pj) + wave * BN;
    floatx16 acc[Cfg::NDB];
#pragma unroll
    for (int db = 0; db < Cfg::NDB; ++db)
      acc[db] = walk_block_mma<T, BN>(tile, hi, lo, cr, u, wave, db, lane);
#pragma unroll
    for (int db = 0; db < Cfg::NDB; ++db) walk_pack_block<T, BN>(tile, acc[db], wave, db, lane);
    walk_store_rows<T, BN>(tile, op, so.sl, tb, limit, col0, Tdim, wave, lane);
  }
}

// ddA[n, p / Q, p % Q] = sum over column tiles of part[n, p / 128, tile, p % 128] for
// positions p < L; the padded slots of the last chunk are set to 0.  One thread per slot.
__global__ __launch_bounds__(256) void dA_reduce_kernel(const float* __restrict__ part,
                                                        float* __restrict__ ddA, int L, int Q, int C,
                                                        int Ci, int ntiles, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t n = i / ((int64_t)C * Q);
  const int64_t p = i - n * (int64_t)C * Q;
  float s = 0.f;
  if (p < L) {
    const int64_t ci = p / kTileRows;
    const int q = (int)(p - ci * kTileRows);
    const float* pp = part + ((n * Ci + ci) * ntiles) * (int64_t)kTileRows + q;
    for (int t = 0; t < ntiles; ++t) s += pp[(int64_t)t * kTileRows];
  }
  ddA[i] = s;
}

}  // namespace ema
