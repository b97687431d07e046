// Single-pass forward and backward of the EMA scan over 128-row chunks.
//
// The carried state that links one chunk to the next is not produced by separate passes
// over x (chunk states, then a sequential recurrence) but inside the one kernel that also
// computes the outputs, by a chained scan with decoupled look-back:
//
//   * every tile (n, chunk c, column tile) publishes the chunk-local state of its columns
//     as soon as it has reduced its rows (flag AGGREGATE), then looks back over the tiles
//     of the earlier chunks of the same sequence and columns, adding decayed aggregates
//     until it meets a tile that already knows its inclusive state (flag PREFIX); it then
//     publishes its own inclusive state and goes on to the MFMA work with the tile still
//     in LDS.  x is read once and y written once.
//   * a published word is 64 bits, {flag, f32 value}, written and polled with relaxed
//     agent-scope atomics, so flag and value arrive together and no fence is needed.
//   * tiles are handed out by an atomic ticket counter in chunk-major order (all columns
//     of chunk 0, then chunk 1, ...; the backward runs the chunks from last to first), so
//     a tile only ever waits for tiles with smaller tickets, which are running or done:
//     the wait cannot deadlock whatever the number of resident workgroups.  Every poll
//     loop is bounded; on exhaustion it raises the error word and the kernel still ends.
//   * workgroups are persistent: while a tile is being processed the loads of the next
//     ticket's tile are already in flight into registers.
#pragma once
#include "ema_walk_kernels.h"

namespace ema {

typedef unsigned long long u64;

#ifdef EMA_TIMING
// Development aid: per-tile phase timestamps into a global buffer (never built into the library).
__device__ long long* g_ema_timing = nullptr;
#define EMA_STAMP(slot)                                                          \
  do {                                                                           \
    if (threadIdx.x == 0 && g_ema_timing) g_ema_timing[(int64_t)cur * 8 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define EMA_STAMP(slot) \
  do {                  \
  } while (0)
#endif

constexpr unsigned kFlagAggregate = 1u;
constexpr unsigned kFlagPrefix = 2u;
constexpr int kSpinLimit = 1 << 20;

__device__ __forceinline__ void chain_publish(u64* p, unsigned flag, float v) {
  const u64 w = ((u64)flag << 32) | (u64)__float_as_uint(v);
  __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Polls one word until it carries a flag.  Gives up after kSpinLimit polls: raises *err and
// reports a zero PREFIX so that the caller's walk ends.
__device__ __forceinline__ unsigned chain_wait(const u64* p, float* v, unsigned* err) {
  for (int i = 0; i < kSpinLimit; ++i) {
    const u64 w = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned f = (unsigned)(w >> 32);
    if (f) {
      *v = __uint_as_float((unsigned)w);
      return f;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  atomicExch(err, 1u);
  *v = 0.f;
  return kFlagPrefix;
}

// Zeroes the status words, the ticket counters and the error word before a chained kernel.
__global__ __launch_bounds__(256) void chain_init_kernel(uint4* __restrict__ words, int64_t n16,
                                                         unsigned* __restrict__ counters) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) words[i] = make_uint4(0u, 0u, 0u, 0u);
  if (i < 4) counters[i] = 0u;
}

struct ChainTile {
  int c, ctile, limit, col0, n, b, h, chunk_id, col_id;  // col_id = n * ntiles + ctile
};

// Ticket -> tile, chunk-major; REV runs the chunks from last to first.  All quantities fit
// 32 bits (the host checks N * C * ntiles < 2^31).
template <bool REV, int BN>
__device__ __forceinline__ ChainTile chain_decode(int ticket, int cols, int ntiles, int C, int nh,
                                                  int L) {
  ChainTile t;
  const unsigned cc = (unsigned)ticket / (unsigned)cols;
  t.c = REV ? C - 1 - (int)cc : (int)cc;
  t.col_id = ticket - (int)cc * cols;
  t.n = (int)((unsigned)t.col_id / (unsigned)ntiles);
  t.ctile = t.col_id - t.n * ntiles;
  t.b = (int)((unsigned)t.n / (unsigned)nh);
  t.h = t.n - t.b * nh;
  t.chunk_id = t.n * C + t.c;
  t.limit = min(kTileRows, L - t.c * kTileRows);
  t.col0 = t.ctile * BN;
  return t;
}

template <typename T, int BN>
__device__ __forceinline__ void chain_issue_loads(Vec16<T>* pre, const T* __restrict__ base,
                                                  SeqStrides s, const ChainTile& t, int Tdim,
                                                  int tid) {
  using C = WalkCfg<T, BN>;
  const T* g = base + (int64_t)t.b * s.sb + (int64_t)t.h * s.sh + (int64_t)t.c * kTileRows * s.sl;
  const int vcol = (tid % C::VPR) * C::EPL;
  const bool cok = t.col0 + vcol < Tdim;
#pragma unroll
  for (int p = 0; p < kTileRows / C::RPP; ++p) {
    const int r = tid / C::VPR + p * C::RPP;
    if (r < t.limit && cok) pre[p] = load16(g + (int64_t)r * s.sl + t.col0 + vcol);
    else pre[p].zero();
  }
}

template <typename T, int BN>
__device__ __forceinline__ void chain_commit_loads(T* tile, const Vec16<T>* pre, int tid) {
  using C = WalkCfg<T, BN>;
  const int vcol = (tid % C::VPR) * C::EPL;
#pragma unroll
  for (int p = 0; p < kTileRows / C::RPP; ++p)
    store16(&tile[(tid / C::VPR + p * C::RPP) * C::ROW + vcol], pre[p]);
}

// State of column t after the chunk when nothing is carried in, and the chunk's total decay.
template <int BN>
__device__ __forceinline__ void chain_local_fwd(const WalkScratch& s, int t, float* loc, float* dec) {
  float l = 0.f, d = 1.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float dj = walk_block_decay(s.csT, j);
    l = fmaf(dj, l, s.sj[j * BN + t]);
    d *= dj;
  }
  *loc = l;
  *dec = d;
}
template <int BN>
__device__ __forceinline__ void chain_local_rev(const WalkScratch& s, int t, float* loc, float* dec) {
  float l = 0.f, d = 1.f;
#pragma unroll
  for (int j = 3; j >= 0; --j) {
    const float dj = walk_block_decay(s.csT, j);
    l = fmaf(dj, l, s.rj[j * BN + t]);
    d *= dj;
  }
  *loc = l;
  *dec = d;
}

// Inclusive state entering chunk c for one column: walks the published words of the chunks
// before (forward) or after (reverse) c.  status points at the words of this column set,
// laid out [chunk][BN]; cs_last(j) is the total log-decay of chunk j.
template <bool REV, int BN>
__device__ __forceinline__ float chain_look(const u64* status, const float* __restrict__ cs_n,
                                            int c, int C, int t, unsigned* err) {
  float carry = 0.f, scale = 1.f;
  for (int j = REV ? c + 1 : c - 1; REV ? j < C : j >= 0; j += REV ? 1 : -1) {
    float v;
    const unsigned f = chain_wait(status + (int64_t)j * BN + t, &v, err);
    carry = fmaf(scale, v, carry);
    if (f == kFlagPrefix) break;
    scale *= __expf(fminf(cs_n[(int64_t)j * kTileRows + kTileRows - 1], 0.f));
  }
  return carry;
}

// ------------------------------------------------------------------------------------
// Forward: y = scan(x) over chunks of 128 rows, one pass.  Also writes prev[n,c,:] (the
// state entering chunk c), optionally a copy at a coarser chunking (every `ratio`-th
// chunk, for callers whose chunk size is a multiple of 128) and the final state.
// status: N*ntiles*C*BN words (zeroed); counters[0] ticket, counters[3] error word.
// ------------------------------------------------------------------------------------
template <typename T, int BN, bool WRITE_Y>
__global__ __launch_bounds__(256, 4) void fwd_chained_kernel(
    const T* __restrict__ x, SeqStrides sx, const float* __restrict__ cs, T* __restrict__ y,
    SeqStrides sy, float* __restrict__ prev, float* __restrict__ prev_coarse, int ratio,
    float* __restrict__ final_state, u64* __restrict__ status, unsigned* __restrict__ counters,
    int nh, int L, int Tdim, int C, int ntiles, int cols, int total) {
  using Cfg = WalkCfg<T, BN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  const WalkScratch s = walk_scratch<T, BN, 1>(smem, 1);
  __shared__ int s_ticket[2];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  unsigned* err = counters + 3;

  if (tid == 0) s_ticket[0] = (int)atomicAdd(counters, 1u);
  __syncthreads();
  int cur = s_ticket[0];
  int slot = 1;
  Vec16<T> pre[kTileRows / Cfg::RPP];
  ChainTile t = chain_decode<false, BN>(cur < total ? cur : 0, cols, ntiles, C, nh, L);
  if (cur < total) chain_issue_loads<T, BN>(pre, x, sx, t, Tdim, tid);
  while (cur < total) {
    EMA_STAMP(0);
    chain_commit_loads<T, BN>(tile, pre, tid);
    walk_load_cs<true, false>(s, cs + (int64_t)t.chunk_id * kTileRows, 0, kTileRows, tid);
    if (tid == 0) s_ticket[slot] = (int)atomicAdd(counters, 1u);
    __syncthreads();
    EMA_STAMP(1);
    const int nxt = s_ticket[slot];
    slot ^= 1;
    const ChainTile tn = chain_decode<false, BN>(nxt < total ? nxt : 0, cols, ntiles, C, nh, L);
    if (nxt < total) chain_issue_loads<T, BN>(pre, x, sx, tn, Tdim, tid);
    walk_block_state<T, BN>(tile, s.wf, s.sj, wave, lane);
    __syncthreads();
    EMA_STAMP(2);
    if (tid < BN) {
      float loc, dec;
      chain_local_fwd<BN>(s, tid, &loc, &dec);
      u64* st = status + (int64_t)t.col_id * C * BN;
      chain_publish(st + (int64_t)t.c * BN + tid, kFlagAggregate, loc);
      const float p_in = chain_look<false, BN>(st, cs + (int64_t)t.n * C * kTileRows, t.c, C, tid, err);
      const float p_out = fmaf(dec, p_in, loc);
      chain_publish(st + (int64_t)t.c * BN + tid, kFlagPrefix, p_out);
      if (t.col0 + tid < Tdim) {
        prev[(int64_t)t.chunk_id * Tdim + t.col0 + tid] = p_in;
        if (prev_coarse && t.c % ratio == 0)
          prev_coarse[((int64_t)t.n * ((C + ratio - 1) / ratio) + t.c / ratio) * Tdim + t.col0 + tid] = p_in;
        if (t.c == C - 1) final_state[(int64_t)t.n * Tdim + t.col0 + tid] = p_out;
      }
      walk_chain_fwd<BN>(s, p_in, tid);
    }
    EMA_STAMP(3);
    __syncthreads();
    EMA_STAMP(4);
    if (WRITE_Y) {
      Vec16<T> hi[Cfg::NG], lo[Cfg::NG];
      walk_decay_frags<T, false>(s.csT, wave, lane, hi, lo);
      const float cm = s.csT[32 * wave + (lane & 31) + 1];
      const float u = __expf(fminf(cm - s.csT[32 * wave], 0.f));
#pragma unroll
      for (int db = 0; db < Cfg::NDB; ++db) {
        const floatx16 acc = walk_block_mma<T, BN>(tile, hi, lo, s.Pj + wave * BN, u, wave, db, lane);
        walk_pack_block<T, BN>(tile, acc, wave, db, lane);
      }
      walk_store_rows<T, BN>(tile, y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl,
                             sy.sl, 0, t.limit, t.col0, Tdim, wave, lane);
    }
    EMA_STAMP(5);
    __syncthreads();
    EMA_STAMP(6);
    cur = nxt;
    t = tn;
  }
}

// ------------------------------------------------------------------------------------
// Backward: dx, the log-decay gradient partials and (WRITE_Y) the recomputed y, one pass
// over x and dy.  prev[n,c,:] (states entering each chunk, from the forward) is an input;
// the reverse state H entering each chunk from the right comes from the chained scan over
// dy, run from the last chunk to the first.  Per tile the arithmetic is that of
// bwd_fused_kernel: dA[m] = exp(A[m]) * <dx[m], y[m-1]>.
// ------------------------------------------------------------------------------------
template <typename T, int BN, bool WRITE_Y>
__global__ __launch_bounds__(256, 2) void bwd_chained_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ cs, const float* __restrict__ prev, T* __restrict__ dx, SeqStrides sdx,
    T* __restrict__ y, SeqStrides sy, float* __restrict__ part, u64* __restrict__ status,
    unsigned* __restrict__ counters, int nh, int L, int Tdim, int C, int ntiles, int cols, int total) {
  using Cfg = WalkCfg<T, BN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* xt = reinterpret_cast<T*>(smem);
  T* dt = xt + Cfg::TILE;
  const WalkScratch s = walk_scratch<T, BN, 2>(smem, 2);
  __shared__ int s_ticket[2];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31;
  unsigned* err = counters + 3;

  if (tid == 0) s_ticket[0] = (int)atomicAdd(counters + 1, 1u);
  __syncthreads();
  int cur = s_ticket[0];
  int slot = 1;
  Vec16<T> pre_x[kTileRows / Cfg::RPP], pre_d[kTileRows / Cfg::RPP];
  float p_pre = 0.f;
  ChainTile t = chain_decode<true, BN>(cur < total ? cur : 0, cols, ntiles, C, nh, L);
  if (cur < total) {
    chain_issue_loads<T, BN>(pre_d, dy, sd, t, Tdim, tid);
    chain_issue_loads<T, BN>(pre_x, x, sx, t, Tdim, tid);
    if (tid < BN && t.col0 + tid < Tdim) p_pre = prev[(int64_t)t.chunk_id * Tdim + t.col0 + tid];
  }
  while (cur < total) {
    EMA_STAMP(0);
    chain_commit_loads<T, BN>(dt, pre_d, tid);
    chain_commit_loads<T, BN>(xt, pre_x, tid);
    const float p_in = p_pre;
    walk_load_cs<true, true>(s, cs + (int64_t)t.chunk_id * kTileRows, 0, kTileRows, tid);
    if (tid == 0) s_ticket[slot] = (int)atomicAdd(counters + 1, 1u);
    __syncthreads();
    EMA_STAMP(1);
    const int nxt = s_ticket[slot];
    slot ^= 1;
    p_pre = 0.f;
    const ChainTile tn = chain_decode<true, BN>(nxt < total ? nxt : 0, cols, ntiles, C, nh, L);
    if (nxt < total) {
      chain_issue_loads<T, BN>(pre_d, dy, sd, tn, Tdim, tid);
      chain_issue_loads<T, BN>(pre_x, x, sx, tn, Tdim, tid);
      if (tid < BN && tn.col0 + tid < Tdim) p_pre = prev[(int64_t)tn.chunk_id * Tdim + tn.col0 + tid];
    }
    walk_block_state<T, BN>(dt, s.wr, s.rj, wave, lane);
    walk_block_state<T, BN>(xt, s.wf, s.sj, wave, lane);
    __syncthreads();
    EMA_STAMP(2);
    if (tid < BN) {
      float loc, dec;
      chain_local_rev<BN>(s, tid, &loc, &dec);
      u64* st = status + (int64_t)t.col_id * C * BN;
      chain_publish(st + (int64_t)t.c * BN + tid, kFlagAggregate, loc);
      const float h_in = chain_look<true, BN>(st, cs + (int64_t)t.n * C * kTileRows, t.c, C, tid, err);
      chain_publish(st + (int64_t)t.c * BN + tid, kFlagPrefix, fmaf(dec, h_in, loc));
      walk_chain_rev<BN>(s, h_in, tid);
      walk_chain_fwd<BN>(s, p_in, tid);
    }
    EMA_STAMP(3);
    __syncthreads();
    EMA_STAMP(4);

    const float cm = s.csT[32 * wave + l32 + 1];
    Vec16<T> fhi[Cfg::NG], flo[Cfg::NG], rhi[Cfg::NG], rlo[Cfg::NG];
    walk_decay_frags<T, true>(s.csT, wave, lane, rhi, rlo);
    walk_decay_frags<T, false>(s.csT, wave, lane, fhi, flo);
    const float ur = __expf(fminf(s.csT[32 * wave + 32] - cm, 0.f));
    const float uf = __expf(fminf(cm - s.csT[32 * wave], 0.f));
    const float* pw = s.Pj + wave * BN;
    float dot = 0.f;
#pragma unroll 1
    for (int db = 0; db < Cfg::NDB; ++db) {
      const floatx16 dacc = walk_block_mma<T, BN>(dt, rhi, rlo, s.Hj + wave * BN, ur, wave, db, lane);
      const floatx16 yacc = walk_block_mma<T, BN>(xt, fhi, flo, pw, uf, wave, db, lane);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float left = __int_as_float(__builtin_amdgcn_update_dpp(
            0, __float_as_int(yacc[v]), 0x138 /* wave_shr:1 */, 0xf, 0xf, false));
        const float ym1 = l32 == 0 ? pw[db * 32 + acc_row(v, lane)] : left;
        dot = fmaf(dacc[v], ym1, dot);
      }
      walk_pack_block<T, BN>(dt, dacc, wave, db, lane);
      if (WRITE_Y) walk_pack_block<T, BN>(xt, yacc, wave, db, lane);
    }
    dot += __shfl_xor(dot, 32);
    if (lane < 32) {
      const int m = 32 * wave + lane;
      part[((int64_t)t.chunk_id * ntiles + t.ctile) * kTileRows + m] =
          m < t.limit ? __expf(cm - s.csT[m]) * dot : 0.f;
    }
    walk_store_rows<T, BN>(dt, dx + (int64_t)t.b * sdx.sb + (int64_t)t.h * sdx.sh + (int64_t)t.c * kTileRows * sdx.sl,
                           sdx.sl, 0, t.limit, t.col0, Tdim, wave, lane);
    if (WRITE_Y)
      walk_store_rows<T, BN>(xt, y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl,
                             sy.sl, 0, t.limit, t.col0, Tdim, wave, lane);
    EMA_STAMP(5);
    __syncthreads();
    EMA_STAMP(6);
    cur = nxt;
    t = tn;
  }
}

}  // namespace ema
