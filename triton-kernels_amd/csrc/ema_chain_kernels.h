// Chained scan with decoupled look-back: what links one 128-row tile of the single-pass
// kernels (ema_tile_kernels.h) to the next.
//
// The carried state is not produced by separate passes over x (chunk states, then a
// sequential recurrence) but inside the one kernel that also computes the outputs:
//
//   * every tile (n, chunk c, column tile) publishes the chunk-local state of its columns
//     as soon as it has reduced its rows (flag AGGREGATE), then looks back over the tiles
//     of the earlier chunks of the same sequence and columns, adding decayed aggregates
//     until it meets a tile that already knows its inclusive state (flag PREFIX); it then
//     publishes its own inclusive state.
//   * a published word is 64 bits, {flag, f32 value}, written and polled with relaxed
//     agent-scope atomics, so flag and value arrive together and no fence is needed.
//   * tiles are handed out by an atomic ticket counter in chunk-major order (all columns
//     of chunk 0, then chunk 1, ...; the backward runs the chunks from last to first), so
//     a tile only ever waits for tiles with smaller tickets, which are running or done:
//     the wait cannot deadlock whatever the number of resident workgroups.  Every poll
//     loop is bounded; on exhaustion it raises the error word and the kernel still ends.
#pragma once
#include "ema_walk_kernels.h"

namespace ema {

typedef unsigned long long u64;

#ifdef EMA_TIMING
// Development aid: per-tile phase timestamps into a global buffer (never built into the library).
__device__ long long* g_ema_timing = nullptr;
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

// Prepares the status words, the ticket counters and the error word before a chained kernel.
// The words of one column set are laid out [slot][BN] with C + 1 slots: C tiles and one
// virtual neighbour before the first tile (forward: slot 0, tiles at slot c + 1) or after the
// last (reverse: slot C, tiles at slot c).  Tile slots are zeroed; the virtual slot carries
// PREFIX with the state that enters the scan from outside, seed[n, column] or 0.  Each thread
// writes two adjacent words (BN is even, so both lie in one slot).
// The set-up of a single-pass kernel in one launch: the first init_blocks workgroups clear the
// status words (and seed the virtual slot), the rest, if any, compute the per-tile cumsum of the
// log-decay that the look-back reads (cumsum_block; cs null = no such workgroups are launched).
// A forward pass whose backward will follow can have the backward's status words prepared in the
// same launch (next: the words of the reverse scan with nothing entering it, next_blocks
// workgroups after the first init_blocks) together with a second copy of the cumsum (cs_next).
struct ChainNext {
  uint4* words;
  int64_t n_pairs;
  unsigned* counters;
  int BN, virt_slot, blocks;
  float* cs;
};
__global__ __launch_bounds__(256) void chain_init_kernel(uint4* __restrict__ words, int64_t n_pairs,
                                                         unsigned* __restrict__ counters, int BN,
                                                         int slots, int virt_slot, int ntiles, int Tdim,
                                                         const float* __restrict__ seed, int init_blocks,
                                                         const float* __restrict__ A, SeqStrides sa,
                                                         float* __restrict__ cs, int nh, int L, int C,
                                                         int64_t total_chunks, int prob, ChainNext next) {
  int64_t blk = blockIdx.x;
  if (blk >= init_blocks + next.blocks) {
    cumsum_block(blk - init_blocks - next.blocks, A, sa, cs, nh, L, kTileRows, C, total_chunks, prob, next.cs);
    return;
  }
  if (blk >= init_blocks) {  // the pass that follows: same layout, its own column width, no seed
    blk -= init_blocks;
    words = next.words, n_pairs = next.n_pairs, counters = next.counters, BN = next.BN;
    virt_slot = next.virt_slot, seed = nullptr;
  }
  const int64_t i = blk * 256 + threadIdx.x;
  if (i < 4) counters[i] = 0u;
  if (i >= n_pairs) return;
  const int64_t w = 2 * i;
  const int64_t row = w / BN;  // (column set, slot)
  const int k = (int)(w - row * BN);
  const int64_t col_id = row / slots;
  const int slot = (int)(row - col_id * slots);
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (slot == virt_slot) {
    float s0 = 0.f, s1 = 0.f;
    if (seed) {
      const int64_t n = col_id / ntiles;
      const int col = (int)(col_id - n * ntiles) * BN + k;
      if (col < Tdim) s0 = seed[n * Tdim + col];
      if (col + 1 < Tdim) s1 = seed[n * Tdim + col + 1];
    }
    v = make_uint4(__float_as_uint(s0), kFlagPrefix, __float_as_uint(s1), kFlagPrefix);
  }
  words[i] = v;
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


// Inclusive state entering chunk c for one column: walks the published words of the chunks
// before (forward) or after (reverse) c, ending at the virtual neighbour at the latest.
// status points at the words of this column set, laid out [slot][BN] as chain_init_kernel
// describes; cs_n[j * 128 + 127] is the total log-decay of chunk j.
template <bool REV, int BN>
__device__ __forceinline__ float chain_look(const u64* status, const float* __restrict__ cs_n,
                                            int c, int C, int t, unsigned* err) {
  float carry = 0.f, scale = 1.f;
  for (int j = REV ? c + 1 : c - 1; REV ? j <= C : j >= -1; j += REV ? 1 : -1) {
    float v;
    const unsigned f = chain_wait(status + (int64_t)(REV ? j : j + 1) * BN + t, &v, err);
    carry = fmaf(scale, v, carry);
    if (f == kFlagPrefix) break;  // always so at the virtual neighbour
    scale *= __expf(fminf(cs_n[(int64_t)j * kTileRows + kTileRows - 1], 0.f));
  }
  return carry;
}

// Slot of tile c of a column set.
template <bool REV>
__device__ __forceinline__ int chain_slot(int c) {
  return REV ? c : c + 1;
}

}  // namespace ema
