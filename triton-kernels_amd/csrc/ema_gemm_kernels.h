// The dy . x^T contraction over the feature axis for the intra-chunk log-decay gradient
// (stage B6 on its own).  bf16 operands use v_mfma_f32_32x32x16_bf16, f32 operands
// v_mfma_f32_32x32x2_f32; accumulation is f32 in both.
#pragma once
#include "ema_device.h"

namespace ema {

constexpr int kBM = 128;  // rows of a chunk handled by one workgroup (4 waves x 32)

// ------------------------------------------------------------------------------------
// B6, first part.  For the chunk (n, c) and the row tile mt (rows m of dy), for every
// column tile kt <= mt (rows k of x):
//   G[m,k] = <dy[m,:], x[k,:]>  (MFMA over the feature axis, operands read row-major)
//   W[m,k] = G[m,k] * exp(min(cs[m]-cs[k],0)) for k < m, else 0; with wk (per-position
//            weights, laid out like cs) and wmk (a (batch, C, ngroups, Q, Q) matrix per chunk
//            and group of heads_per_group heads) also * wk[k] * wmk[m,k]: the form the SSD
//            scan needs (wk = dt, wmk = C B^T); both are null for the EMA scan
//   part[(chunk*MT + mt)*Q + k] = sum_m W[m,k]      (column sums of this row tile)
//   rowsum[chunk*Q + m]         = sum_k W[m,k]      (complete: all k < m are visited)
// da_finish_kernel turns these into ddA_intra.
// ------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256, 2) void da_gemm_kernel(const T* __restrict__ x, SeqStrides sx,
                                                      const T* __restrict__ dy, SeqStrides sd,
                                                      const float* __restrict__ cs,
                                                      float* __restrict__ part,
                                                      float* __restrict__ rowsum, int nh, int L,
                                                      int Tdim, int Q, int C, int MT,
                                                      const float* __restrict__ wk,
                                                      const float* __restrict__ wmk,
                                                      int heads_per_group, int ngroups,
                                                      const int* __restrict__ only = nullptr) {
  // only (may be null): the kernel works on the chunks whose entry is not 0 and leaves the rest alone
  if (only && only[blockIdx.x / MT] == 0) return;
  constexpr int EPL = Vec16<T>::N;
  constexpr int KG = 2 * EPL;
  constexpr int DK = 4 * KG;        // feature columns per LDS stage (128 bytes per row)
  constexpr int ROW = DK + EPL;     // row pitch in elements (16 bytes of padding)
  constexpr int TILE = kBM * ROW;   // elements per staged tile
  // staging tiles, later reused for the row-sum exchange (256 x 17 floats = 17408 bytes)
  __shared__ __attribute__((aligned(16))) T stage[2 * TILE];
  __shared__ float cs_s[EMA_MAX_CHUNK_DEV];
  __shared__ float colpart[4 * 2 * kBM];
  static_assert(2 * TILE * sizeof(T) >= 256 * 17 * sizeof(float), "row exchange must fit");
  T* dys = stage;
  T* xs = stage + TILE;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int mt = (int)(blockIdx.x % MT);
  const int64_t chunk_id = blockIdx.x / MT;
  const int64_t n = chunk_id / C;
  const int c = (int)(chunk_id - n * C);
  const int64_t b = n / nh;
  const int h = (int)(n - b * nh);
  const int limit = min(Q, L - c * Q);
  const int mt_base = mt * kBM;

  const float* csp = cs + chunk_id * Q;
  const float* wkp = wk ? wk + chunk_id * Q : nullptr;
  const float* wmp = wmk ? wmk + (((b * C + c) * ngroups + h / heads_per_group) * (int64_t)Q) * Q : nullptr;
  const int q_pad = (Q + kBM - 1) / kBM * kBM;
  for (int i = tid; i < q_pad; i += 256) cs_s[i] = i < Q ? csp[i] : 0.f;

  const T* xp = x + b * sx.sb + h * sx.sh + (int64_t)c * Q * sx.sl;
  const T* dp = dy + b * sd.sb + h * sd.sh + (int64_t)c * Q * sd.sl;

  float rowacc[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) rowacc[v] = 0.f;

  constexpr int VPR = DK / EPL;   // 8 vectors per row
  constexpr int RPP = 256 / VPR;  // 32 rows per pass
  constexpr int NP = kBM / RPP;   // passes (row pieces per thread and operand)
  const int vcol = (tid % VPR) * EPL;
  const int r0 = tid / VPR;
  // One stage of both operands in registers: requested before the products of the stage before
  // are formed, so that the loads travel meanwhile (the LDS tiles themselves are single).
  Vec16<T> pd[NP], px[NP];
  auto request = [&](int kt_base, int d0) {
    const bool cok = d0 + vcol < Tdim;
    const int dcol = cok ? d0 + vcol : 0;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      // unconditional loads from indices clamped into the tensor, zeroed afterwards
      const int m = mt_base + r0 + p * RPP, k = kt_base + r0 + p * RPP;
      pd[p] = load16(dp + (int64_t)min(m, limit - 1) * sd.sl + dcol);
      px[p] = load16(xp + (int64_t)min(k, limit - 1) * sx.sl + dcol);
      if (m >= limit || !cok) pd[p].zero();
      if (k >= limit || !cok) px[p].zero();
    }
  };
  request(0, 0);
  for (int kt = 0; kt <= mt; ++kt) {
    const int kt_base = kt * kBM;
    const int ncb = kt == mt ? wave + 1 : 4;  // column blocks at or below the diagonal
    floatx16 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[cb][v] = 0.f;

    for (int d0 = 0; d0 < Tdim; d0 += DK) {
      __syncthreads();
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        store16(&dys[(r0 + p * RPP) * ROW + vcol], pd[p]);
        store16(&xs[(r0 + p * RPP) * ROW + vcol], px[p]);
      }
      __syncthreads();
      // the stage after this one: next feature columns, or the first ones of the next column tile
      if (d0 + DK < Tdim) request(kt_base, d0 + DK);
      else if (kt < mt) request(kt_base + kBM, 0);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int doff = g * KG + EPL * half;
        const Vec16<T> a = load16(&dys[(wave * 32 + l32) * ROW + doff]);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
          if (cb < ncb) {
            const Vec16<T> bf = load16(&xs[(cb * 32 + l32) * ROW + doff]);
            mma_group(a, bf, acc[cb]);
          }
        }
      }
    }

    // scale, mask, and reduce this (mt, kt) tile
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
      float colacc = 0.f;
      if (cb < ncb) {
        const int k = kt_base + cb * 32 + l32;
        const float cs_k = cs_s[k];
        const float wk_k = (wkp && k < Q) ? wkp[k] : 1.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = mt_base + wave * 32 + acc_row(v, lane);
          float w = acc[cb][v] * __expf(fminf(cs_s[m] - cs_k, 0.f)) * wk_k;
          // the load is unconditional (row and column clamped into the matrix) so that the
          // sixteen of a block are in flight together
          if (wmp) w *= wmp[(int64_t)min(m, Q - 1) * Q + min(k, Q - 1)];
          w = (k < m && m < limit) ? w : 0.f;
          rowacc[v] += w;
          colacc += w;
        }
      }
      colpart[(wave * 2 + half) * kBM + cb * 32 + l32] = colacc;
    }
    __syncthreads();
    if (tid < kBM) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s += colpart[i * kBM + tid];
      const int k = kt_base + tid;
      if (k < Q) part[(chunk_id * MT + mt) * (int64_t)Q + k] = s;
    }
  }

  __syncthreads();
  float* rowbuf = reinterpret_cast<float*>(stage);
#pragma unroll
  for (int v = 0; v < 16; ++v) rowbuf[tid * 17 + v] = rowacc[v];
  __syncthreads();
  if (tid < kBM) {
    const int w = tid >> 5, rr = tid & 31;
    const int v = 4 * (rr >> 3) + (rr & 3);
    const int hf = (rr >> 2) & 1;
    float s = 0.f;
    for (int l = 0; l < 32; ++l) s += rowbuf[(w * 64 + hf * 32 + l) * 17 + v];
    const int m = mt_base + tid;
    if (m < Q) rowsum[chunk_id * Q + m] = s;
  }
}

// B6, second part: ddA_intra[j] = sum_{i<j} (colsum[i] - rowsum[i]) with
// colsum[i] = sum over the row tiles mt >= i / 128 of part[mt][i].  One wave per (n, c).
// only (may be null): the chunks whose entry is 0 are left alone.
template <int BM>
__global__ __launch_bounds__(256) void da_finish_kernel(const float* __restrict__ part,
                                                        const float* __restrict__ rowsum,
                                                        float* __restrict__ ddA_intra, int Q,
                                                        int MT, int64_t total_chunks,
                                                        const int* __restrict__ only = nullptr) {
  const int lane = threadIdx.x & 63;
  const int64_t chunk_id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk_id >= total_chunks) return;
  if (only && only[chunk_id] == 0) return;
  const int per = (Q + 63) >> 6;
  const int q0 = lane * per;
  auto val = [&](int q) {
    float s = -rowsum[chunk_id * Q + q];
    for (int mt = q / BM; mt < MT; ++mt) s += part[(chunk_id * MT + mt) * (int64_t)Q + q];
    return s;
  };
  float local = 0.f;
  for (int i = 0; i < per; ++i)
    if (q0 + i < Q) local += val(q0 + i);
  float run = wave_inclusive_scan(local) - local;
  for (int i = 0; i < per; ++i) {
    const int q = q0 + i;
    if (q < Q) {
      ddA_intra[chunk_id * Q + q] = run;
      run += val(q);
    }
  }
}

// The same for the factored form, whose per-column-tile dots only have to be added up:
// ddA_intra[chunk][q] = sum over the ntiles column tiles of flat[(chunk*ntiles + tile)*Q + q], for
// the chunks whose entry in steep is 0.  One thread per (chunk, q).
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void da_flat_finish_kernel(const float* __restrict__ flat,
                                                             const int* __restrict__ steep,
                                                             float* __restrict__ ddA_intra, int Q,
                                                             int ntiles, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= total) return;
  const int64_t chunk_id = i / Q;
  if (steep[chunk_id] != 0) return;
  const int q = (int)(i - chunk_id * Q);
  float s = 0.f;
  for (int ct = 0; ct < ntiles; ++ct) s += flat[(chunk_id * ntiles + ct) * (int64_t)Q + q];
  ddA_intra[i] = s;
}

}  // namespace ema
