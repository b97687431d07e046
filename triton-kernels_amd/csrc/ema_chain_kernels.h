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
//     ticket's tile are already in flight into registers, and the ticket after that is
//     being fetched.
//   * per tile, the diagonal-block products (which need no carried state) run first; the
//     chunk-local state is read off their accumulators (the scan value at the last row of a
//     block IS that block's state), published, and only then does the tile wait for the
//     states of its neighbours, whose latency the products have already covered.
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

// Thread layout of a chained kernel: NT threads = NT/64 waves; wave w works on the 32-row
// block w / CH and on the column slice w % CH of the tile, CH = NT / 256.
template <typename T, int BN, int NT>
struct ChainCfg {
  using W = WalkCfg<T, BN>;
  static constexpr int CH = NT / 256;                 // column slices per row block
  static constexpr int RPP = NT / W::VPR;             // rows staged per pass
  static constexpr int NPRE = kTileRows / RPP;        // 16-byte loads per thread and tile
  static constexpr int CW = BN / CH;                  // columns of one wave
  static constexpr int NDBW = W::NDB / CH;            // 32-column blocks per wave
  static_assert(NT == 256 || NT == 512, "4 or 8 waves");
  static_assert(NDBW >= 1 && NPRE >= 1, "tile too narrow for this thread count");
};

// Global addresses of a tile are formed as (uniform base of the row group) + (32-bit lane
// offset), which costs one address register per thread instead of two per load; the host
// refuses row strides for which 128 rows would not fit 32 bits.
template <typename T, int BN, int NT>
__device__ __forceinline__ void chain_issue_loads(Vec16<T>* pre, const T* __restrict__ base,
                                                  SeqStrides s, const ChainTile& t, int Tdim,
                                                  int tid) {
  using C = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  const T* g = base + (int64_t)t.b * s.sb + (int64_t)t.h * s.sh + (int64_t)t.c * kTileRows * s.sl + t.col0;
  const int r0 = tid / C::VPR;
  const unsigned vcol = (unsigned)(tid % C::VPR) * C::EPL;
  const unsigned off = (unsigned)r0 * (unsigned)s.sl + vcol;
  const bool cok = t.col0 + (int)vcol < Tdim;
#pragma unroll
  for (int p = 0; p < CC::NPRE; ++p) {
    const T* gp = g + (int64_t)(p * CC::RPP) * s.sl;  // uniform
    if (r0 + p * CC::RPP < t.limit && cok) pre[p] = load16(gp + off);
    else pre[p].zero();
  }
}

template <typename T, int BN, int NT>
__device__ __forceinline__ void chain_commit_loads(T* tile, const Vec16<T>* pre, int tid) {
  using C = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  const int vcol = (tid % C::VPR) * C::EPL;
#pragma unroll
  for (int p = 0; p < CC::NPRE; ++p)
    store16(&tile[(tid / C::VPR + p * CC::RPP) * C::ROW + vcol], pre[p]);
}

// Rows of block blk, columns of slice ch, from an LDS tile to global memory (16 bytes per
// lane).  g points at (row 0 of the chunk, first column of the tile).
template <typename T, int BN, int NT>
__device__ __forceinline__ void chain_store_rows(const T* tile, T* __restrict__ g, int64_t sl,
                                                 int limit, int col0, int Tdim, int blk, int ch,
                                                 int lane) {
  using C = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  constexpr int VPRH = CC::CW / C::EPL;  // vectors per half row
  constexpr int RPW = 64 / VPRH;         // rows per pass of one wave
  const unsigned vcol = (unsigned)(ch * CC::CW + (lane % VPRH) * C::EPL);
  if (col0 + (int)vcol >= Tdim) return;
  const int r0 = lane / VPRH;
  const unsigned off = (unsigned)r0 * (unsigned)sl + vcol;
#pragma unroll
  for (int p = 0; p < 32 / RPW; ++p) {
    const int r = blk * 32 + p * RPW + r0;
    T* gp = g + (int64_t)(blk * 32 + p * RPW) * sl;  // uniform
    if (r < limit) store16(gp + off, load16(&tile[r * C::ROW + vcol]));
  }
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

// Diagonal-block products of wave (blk, ch) for its NDBW 32-column blocks, without any
// carried state: register v of lane l of acc[d2] is out[row 32 blk + l%32][column
// (ch*NDBW + d2)*32 + 8*(v/4) + 4*(l/32) + v%4].  The decay block is built one MFMA group
// (KG values of k) at a time and used at once for every column block, so that only one
// group of factors is live.
//   forward: (k <= m) * exp(cs[m] - cs[k]);  reverse: (k >= m) * exp(cs[k] - cs[m]),
// split as bf16 hi + lo for bf16 operands.
template <typename T, int BN, int NT, bool REV>
__device__ __forceinline__ void chain_local_products(const T* tile, const float* csT, int blk, int ch,
                                                     int lane, floatx16* acc) {
  using C = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  constexpr int EPL = C::EPL;
  const int rm = 32 * blk + (lane & 31);
  const float cm = csT[rm + 1];
#pragma unroll
  for (int d2 = 0; d2 < CC::NDBW; ++d2)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[d2][v] = 0.f;
#pragma unroll
  for (int g = 0; g < C::NG; ++g) {
    Vec16<T> hi, lo;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int k = 32 * blk + g * C::KG + EPL * (lane >> 5) + e;
      const float ck = csT[k + 1];
      const bool keep = REV ? (k >= rm) : (k <= rm);
      // branch-free: a masked element gets exp(-huge) = 0
      const float val = __expf(keep ? fminf(REV ? ck - cm : cm - ck, 0.f) : -1.0e30f);
      hi.set(e, val);
      if (sizeof(T) == 2) lo.set(e, val - hi.get(e));
    }
#pragma unroll
    for (int d2 = 0; d2 < CC::NDBW; ++d2) {
      const int db = ch * CC::NDBW + d2;
      const Vec16<T> xf = walk_in_frag(tile, C::ROW, 32 * blk + g * C::KG, db * 32, lane);
      mma_group(xf, hi, acc[d2]);
      if (sizeof(T) == 2) mma_group(xf, lo, acc[d2]);
    }
  }
}

// The lanes that hold row `row32` of the block (one lane per half-wave) write their 16
// accumulators, times `scale`, to out[db*32 + column]: a block's local state.
__device__ __forceinline__ void chain_extract_row(float* out, const floatx16& acc, float scale,
                                                  int row32, int db, int lane) {
  if ((lane & 31) == row32) {
    float* p = out + db * 32 + 4 * (lane >> 5);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4*>(p + 8 * q) = make_float4(scale * acc[4 * q + 0], scale * acc[4 * q + 1],
                                                           scale * acc[4 * q + 2], scale * acc[4 * q + 3]);
  }
}

// acc += u * carry[column]; returns the four carry vectors read (the caller may need them).
__device__ __forceinline__ void chain_add_carry(floatx16& acc, float4* c4, const float* carry,
                                                float u, int db, int lane) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    c4[q] = *reinterpret_cast<const float4*>(&carry[db * 32 + 8 * q + 4 * (lane >> 5)]);
    acc[4 * q + 0] = fmaf(u, c4[q].x, acc[4 * q + 0]);
    acc[4 * q + 1] = fmaf(u, c4[q].y, acc[4 * q + 1]);
    acc[4 * q + 2] = fmaf(u, c4[q].z, acc[4 * q + 2]);
    acc[4 * q + 3] = fmaf(u, c4[q].w, acc[4 * q + 3]);
  }
}

// Ticket bookkeeping of a persistent workgroup: `cur` is being processed, `nxt` is
// prefetched, and the one after is requested at the top of an iteration and collected at
// its end, so that no iteration waits for the atomic.
struct ChainTickets {
  int cur, nxt;
};
__device__ __forceinline__ ChainTickets chain_first_tickets(unsigned* counter, int* s_ticket, int tid) {
  if (tid == 0) {
    s_ticket[0] = (int)atomicAdd(counter, 1u);
    s_ticket[1] = (int)atomicAdd(counter, 1u);
  }
  __syncthreads();
  ChainTickets t;
  t.cur = s_ticket[0];
  t.nxt = s_ticket[1];
  __syncthreads();
  return t;
}

// ------------------------------------------------------------------------------------
// Forward: y = scan(x) over chunks of 128 rows, one pass.  Also writes prev[n,c,:] (the
// state entering chunk c), optionally a copy at a coarser chunking (every `ratio`-th
// chunk, for callers whose chunk size is a multiple of 128) and the final state.
// status: N*ntiles*C*BN words (zeroed); counters[0] ticket, counters[3] error word.
// ------------------------------------------------------------------------------------
template <typename T, int BN, int NT, int MINW, bool WRITE_Y>
__global__ __launch_bounds__(NT, MINW) void fwd_chained_kernel(
    const T* __restrict__ x, SeqStrides sx, const float* __restrict__ cs, T* __restrict__ y,
    SeqStrides sy, float* __restrict__ prev, float* __restrict__ prev_coarse, int ratio,
    float* __restrict__ final_state, u64* __restrict__ status, unsigned* __restrict__ counters,
    int nh, int L, int Tdim, int C, int ntiles, int cols, int total) {
  using Cfg = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  const WalkScratch s = walk_scratch<T, BN, 1>(smem, 1);
  __shared__ int s_ticket[2];

  const int tid0 = threadIdx.x;
  const int blk = (tid0 >> 6) / CC::CH, ch = (tid0 >> 6) % CC::CH;  // row block, column slice of this wave
  unsigned* err = counters + 3;

  ChainTickets tk = chain_first_tickets(counters, s_ticket, tid0);
  int tid = tid0;
  int cur = tk.cur, nxt = tk.nxt;
  Vec16<T> pre[CC::NPRE];
  ChainTile t = chain_decode<false, BN>(cur < total ? cur : 0, cols, ntiles, C, nh, L);
  if (cur < total) chain_issue_loads<T, BN, NT>(pre, x, sx, t, Tdim, tid);
  while (cur < total) {
    // The thread index is made opaque once per tile so that the many per-lane addresses and
    // masks derived from it are recomputed per tile instead of being kept in registers for
    // the whole persistent loop.
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, l32 = lane & 31;
    EMA_STAMP(0);
    chain_commit_loads<T, BN, NT>(tile, pre, tid);
    const ChainTile tn = chain_decode<false, BN>(nxt < total ? nxt : 0, cols, ntiles, C, nh, L);
    if (nxt < total) chain_issue_loads<T, BN, NT>(pre, x, sx, tn, Tdim, tid);
    int future = 0;
    if (tid == 0) future = (int)atomicAdd(counters, 1u);
    walk_load_cs<false, false>(s, cs + (int64_t)t.chunk_id * kTileRows, 0, kTileRows, tid);
    __syncthreads();
    EMA_STAMP(1);

    // local products; the block's state is the local scan value at its last row
    floatx16 acc[CC::NDBW];
    chain_local_products<T, BN, NT, false>(tile, s.csT, blk, ch, lane, acc);
#pragma unroll
    for (int d2 = 0; d2 < CC::NDBW; ++d2)
      chain_extract_row(s.sj + blk * BN, acc[d2], 1.f, 31, ch * CC::NDBW + d2, lane);
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
      const float cm = s.csT[32 * blk + l32 + 1];
      const float u = __expf(fminf(cm - s.csT[32 * blk], 0.f));
#pragma unroll
      for (int d2 = 0; d2 < CC::NDBW; ++d2) {
        const int db = ch * CC::NDBW + d2;
        float4 c4[4];
        chain_add_carry(acc[d2], c4, s.Pj + blk * BN, u, db, lane);
        walk_pack_block<T, BN>(tile, acc[d2], blk, db, lane);
      }
      chain_store_rows<T, BN, NT>(tile, y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl + t.col0,
                              sy.sl, t.limit, t.col0, Tdim, blk, ch, lane);
    }
    EMA_STAMP(5);
    if (tid == 0) s_ticket[0] = future;
    __syncthreads();
    EMA_STAMP(6);
    cur = nxt;
    nxt = s_ticket[0];
    t = tn;
  }
}

// ------------------------------------------------------------------------------------
// Backward: dx, the log-decay gradient partials and (WRITE_Y) the recomputed y, one pass
// over x and dy.  prev[n,c,:] (states entering each chunk, from the forward) is an input;
// the reverse state H entering each chunk from the right comes from the chained scan over
// dy, run from the last chunk to the first.  Per tile:
//   dx[m] = local + exp(cs[e]-cs[m]) * H,   y[m] = local + exp(cs[m]-cs[s]) * P,
//   dA[m] = exp(A[m]) * <dx[m], y[m-1]>     (y[-1] of a block is its carried state P),
// reduced over the columns of each wave into part[((chunk*ntiles + ctile)*CH + slice)*128 + m].
// ------------------------------------------------------------------------------------
template <typename T, int BN, int NT, int MINW, bool WRITE_Y>
__global__ __launch_bounds__(NT, MINW) void bwd_chained_kernel(
    const T* __restrict__ x, SeqStrides sx, const T* __restrict__ dy, SeqStrides sd,
    const float* __restrict__ cs, const float* __restrict__ prev, T* __restrict__ dx, SeqStrides sdx,
    T* __restrict__ y, SeqStrides sy, float* __restrict__ part, u64* __restrict__ status,
    unsigned* __restrict__ counters, int nh, int L, int Tdim, int C, int ntiles, int cols, int total) {
  using Cfg = WalkCfg<T, BN>;
  using CC = ChainCfg<T, BN, NT>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* xt = reinterpret_cast<T*>(smem);
  T* dt = xt + Cfg::TILE;
  const WalkScratch s = walk_scratch<T, BN, 2>(smem, 2);
  __shared__ int s_ticket[2];

  const int tid0 = threadIdx.x;
  const int blk = (tid0 >> 6) / CC::CH, ch = (tid0 >> 6) % CC::CH;  // row block, column slice of this wave
  unsigned* err = counters + 3;

  ChainTickets tk = chain_first_tickets(counters + 1, s_ticket, tid0);
  int tid = tid0;
  int cur = tk.cur, nxt = tk.nxt;
  Vec16<T> pre_x[CC::NPRE], pre_d[CC::NPRE];
  float p_pre = 0.f;
  ChainTile t = chain_decode<true, BN>(cur < total ? cur : 0, cols, ntiles, C, nh, L);
  if (cur < total) {
    chain_issue_loads<T, BN, NT>(pre_d, dy, sd, t, Tdim, tid);
    chain_issue_loads<T, BN, NT>(pre_x, x, sx, t, Tdim, tid);
    if (tid < BN && t.col0 + tid < Tdim) p_pre = prev[(int64_t)t.chunk_id * Tdim + t.col0 + tid];
  }
  while (cur < total) {
    asm volatile("" : "+v"(tid));  // see fwd_chained_kernel
    const int lane = tid & 63, l32 = lane & 31;
    EMA_STAMP(0);
    chain_commit_loads<T, BN, NT>(dt, pre_d, tid);
    chain_commit_loads<T, BN, NT>(xt, pre_x, tid);
    const float p_in = p_pre;
    const ChainTile tn = chain_decode<true, BN>(nxt < total ? nxt : 0, cols, ntiles, C, nh, L);
    int future = 0;
    if (tid == 0) future = (int)atomicAdd(counters + 1, 1u);
    walk_load_cs<false, false>(s, cs + (int64_t)t.chunk_id * kTileRows, 0, kTileRows, tid);
    __syncthreads();
    EMA_STAMP(1);

    // local products in both directions; block states read off the accumulators
    floatx16 dacc[CC::NDBW], yacc[CC::NDBW];
    chain_local_products<T, BN, NT, true>(dt, s.csT, blk, ch, lane, dacc);
    {
      // local reverse state referenced to the row before the block: exp(A[first]) * dx_local[first]
      const float ea = __expf(fminf(s.csT[32 * blk + 1] - s.csT[32 * blk], 0.f));
#pragma unroll
      for (int d2 = 0; d2 < CC::NDBW; ++d2)
        chain_extract_row(s.rj + blk * BN, dacc[d2], ea, 0, ch * CC::NDBW + d2, lane);
    }
    chain_local_products<T, BN, NT, false>(xt, s.csT, blk, ch, lane, yacc);
#pragma unroll
    for (int d2 = 0; d2 < CC::NDBW; ++d2)
      chain_extract_row(s.sj + blk * BN, yacc[d2], 1.f, 31, ch * CC::NDBW + d2, lane);
    // the next tile's loads start here rather than at the top of the iteration: they stay
    // in flight through the look-back and the finishing phase, and their registers are not
    // live while both sets of accumulators are being built
    p_pre = 0.f;
    if (nxt < total) {
      chain_issue_loads<T, BN, NT>(pre_d, dy, sd, tn, Tdim, tid);
      chain_issue_loads<T, BN, NT>(pre_x, x, sx, tn, Tdim, tid);
      if (tid < BN && tn.col0 + tid < Tdim) p_pre = prev[(int64_t)tn.chunk_id * Tdim + tn.col0 + tid];
    }
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

    const float cm = s.csT[32 * blk + l32 + 1];
    const float ur = __expf(fminf(s.csT[32 * blk + 32] - cm, 0.f));
    const float uf = __expf(fminf(cm - s.csT[32 * blk], 0.f));
    float dot = 0.f;
#pragma unroll
    for (int d2 = 0; d2 < CC::NDBW; ++d2) {
      const int db = ch * CC::NDBW + d2;
      // carried states in; y[m-1] sits one lane to the left, and the block's first row takes
      // the carried state P itself
      float dsum[4] = {0.f, 0.f, 0.f, 0.f};
      const float* hp = s.Hj + blk * BN + db * 32 + 4 * (lane >> 5);
      const float* pp = s.Pj + blk * BN + db * 32 + 4 * (lane >> 5);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 h4 = *reinterpret_cast<const float4*>(hp + 8 * q);
        const float4 p4 = *reinterpret_cast<const float4*>(pp + 8 * q);
        const float hv[4] = {h4.x, h4.y, h4.z, h4.w};
        const float pv[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int v = 4 * q + i;
          dacc[d2][v] = fmaf(ur, hv[i], dacc[d2][v]);
          yacc[d2][v] = fmaf(uf, pv[i], yacc[d2][v]);
          const float left = __int_as_float(__builtin_amdgcn_update_dpp(
              0, __float_as_int(yacc[d2][v]), 0x138 /* wave_shr:1 */, 0xf, 0xf, false));
          dsum[i] = fmaf(dacc[d2][v], l32 == 0 ? pv[i] : left, dsum[i]);
        }
      }
      dot += (dsum[0] + dsum[1]) + (dsum[2] + dsum[3]);
      walk_pack_block<T, BN>(dt, dacc[d2], blk, db, lane);
      if (WRITE_Y) walk_pack_block<T, BN>(xt, yacc[d2], blk, db, lane);
    }
    dot += __shfl_xor(dot, 32);
    if (lane < 32) {
      const int m = 32 * blk + lane;
      part[(((int64_t)t.chunk_id * ntiles + t.ctile) * CC::CH + ch) * kTileRows + m] =
          m < t.limit ? __expf(cm - s.csT[m]) * dot : 0.f;
    }
    chain_store_rows<T, BN, NT>(dt, dx + (int64_t)t.b * sdx.sb + (int64_t)t.h * sdx.sh + (int64_t)t.c * kTileRows * sdx.sl + t.col0,
                            sdx.sl, t.limit, t.col0, Tdim, blk, ch, lane);
    if (WRITE_Y)
      chain_store_rows<T, BN, NT>(xt, y + (int64_t)t.b * sy.sb + (int64_t)t.h * sy.sh + (int64_t)t.c * kTileRows * sy.sl + t.col0,
                              sy.sl, t.limit, t.col0, Tdim, blk, ch, lane);
    EMA_STAMP(5);
    if (tid == 0) s_ticket[0] = future;
    __syncthreads();
    EMA_STAMP(6);
    cur = nxt;
    nxt = s_ticket[0];
    t = tn;
  }
}

}  // namespace ema
