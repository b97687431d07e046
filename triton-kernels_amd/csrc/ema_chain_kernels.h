// Chained scan with decoupled look-back: what links one 128-row tile of the single-pass
// kernels (ema_tile_kernels.h) to the next.
//
// The carried state is not produced by separate passes over x (chunk states, then a
// sequential recurrence) but inside the one kernel that also computes the outputs:
//
//   * every tile (n, chunk c, column tile) publishes the chunk-local state of its columns
//     as soon as it has reduced its rows (state AGGREGATE) together with the tile's total
//     decay, then looks back over the tiles of the earlier chunks of the same sequence and
//     columns, adding decayed aggregates until it meets a tile that already knows its
//     inclusive state (state PREFIX); it then publishes its own inclusive state.
//   * a published word is 64 bits, {tag, f32 value}, written and polled with relaxed
//     agent-scope atomics, so tag and value arrive together and no fence is needed.
//   * the tag holds the launch's epoch besides the state, so words left by earlier launches
//     read as "not published" and nothing has to be cleared between launches: a workspace that
//     was zero-filled once serves any number of launches of any shapes, one after the other.
//     The header of the workspace carries the epoch; the last workgroup to leave a launch
//     advances it and puts the ticket counter back to zero.
//   * tiles are handed out by an atomic ticket counter in chunk-major order (all columns
//     of chunk 0, then chunk 1, ...; the backward runs the chunks from last to first), so
//     a tile only ever waits for tiles with smaller tickets, which are running or done:
//     the wait cannot deadlock whatever the number of resident workgroups.  Every poll
//     loop is bounded; on exhaustion it raises the error word of the header, hands on NaN
//     (which reaches the outputs) and the kernel still ends.
#pragma once
#include "ema_walk_kernels.h"

namespace ema {

typedef unsigned long long u64;

#ifdef EMA_TIMING
// Development aid: per-tile phase timestamps into a global buffer (never built into the library).
__device__ long long* g_ema_timing = nullptr;
#endif

// First 256 bytes of a chained-scan workspace (ema_chain_header in ema_hip.h).
struct ChainHeader {
  unsigned ticket;      // next tile to hand out; zero between launches
  unsigned done;        // workgroups that have left the running launch; zero between launches
  unsigned epoch;       // epoch of the last completed launch
  unsigned error;       // sticky: a bounded wait ran out in some launch since the last clear
  unsigned spin_limit;  // polls before a wait gives up; 0 = kSpinLimitDefault
  unsigned reserved[59];
};
static_assert(sizeof(ChainHeader) == 256, "header size is part of the ABI");

constexpr unsigned kStateAggregate = 1u;
constexpr unsigned kStatePrefix = 2u;
constexpr unsigned kSpinLimitDefault = 1u << 20;
constexpr unsigned kEpochMask = 0x3fffffffu;

// Epoch of the launch that finds `last` in the header: 1 .. 2^30 - 1, never 0 (the tag of
// zero-filled memory).
__device__ __forceinline__ unsigned chain_next_epoch(unsigned last) {
  const unsigned e = (last + 1u) & kEpochMask;
  return e ? e : 1u;
}

__device__ __forceinline__ void chain_publish(u64* p, unsigned epoch, unsigned state, float v) {
  const u64 w = ((u64)((epoch << 2) | state) << 32) | (u64)__float_as_uint(v);
  __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ u64 chain_peek(const u64* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// State of a word under this launch's epoch; 0 = not published by this launch.
__device__ __forceinline__ unsigned chain_state(u64 w, unsigned epoch) {
  const unsigned tag = (unsigned)(w >> 32);
  return (tag >> 2) == epoch ? (tag & 3u) : 0u;
}

__device__ __forceinline__ float chain_value(u64 w) { return __uint_as_float((unsigned)w); }

struct ChainCtl {
  unsigned epoch, spin_limit;
  unsigned* err;
};

// w is what a first look at *p returned.  Polls until the word is published by this launch.
// Gives up after spin_limit polls: raises the error word and reports a PREFIX of NaN, which ends
// the caller's walk and poisons everything computed from it.
__device__ __forceinline__ u64 chain_wait(const u64* p, u64 w, const ChainCtl& ctl) {
  unsigned polls = 0;
  while (chain_state(w, ctl.epoch) == 0u) {
    if (++polls > ctl.spin_limit) {
      atomicExch(ctl.err, 1u);
      return ((u64)((ctl.epoch << 2) | kStatePrefix) << 32) | 0x7fc00000ull;
    }
    __builtin_amdgcn_s_sleep(1);
    w = chain_peek(p);
  }
  return w;
}

// Start and end of a launch.  Every workgroup reads the epoch before its first tile; the last
// one to leave (all tickets are taken by then and nobody reads the header again) advances the
// epoch and zeroes the counters for the next launch on the stream.
__device__ __forceinline__ ChainCtl chain_enter(ChainHeader* hdr) {
  ChainCtl ctl;
  ctl.epoch = chain_next_epoch(__hip_atomic_load(&hdr->epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  const unsigned lim = __hip_atomic_load(&hdr->spin_limit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  ctl.spin_limit = lim ? lim : kSpinLimitDefault;
  ctl.err = &hdr->error;
  return ctl;
}
__device__ __forceinline__ void chain_leave(ChainHeader* hdr, const ChainCtl& ctl) {
  // called by one thread per workgroup after the workgroup's last tile
  const unsigned before = __hip_atomic_fetch_add(&hdr->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (before == gridDim.x - 1) {
    __hip_atomic_store(&hdr->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&hdr->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&hdr->epoch, ctl.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Zero fill of a workspace (or of its leading part) in 16-byte pieces: the state in which the
// chained kernels expect to find a workspace they have not used before.
__global__ __launch_bounds__(256) void chain_clear_kernel(uint4* __restrict__ p, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

// n / d for n < 2^31 by a multiplication: m = ceil(2^(31 + l) / d), l = ceil(log2 d), fits 32 bits
// and floor(n * m / 2^(31 + l)) is exact for n < 2^31 (the error term n * (m * d - 2^(31 + l)) stays
// below 2^(31 + l)).  d = 1 is encoded as m = 0.
struct FastDiv {
  unsigned m, sh;
};
inline FastDiv fast_div_make(unsigned d) {
  FastDiv f{0u, 0u};
  if (d <= 1u) return f;
  unsigned l = 0;
  while ((1ull << l) < d) ++l;
  const unsigned long long num = 1ull << (31 + l);
  f.m = (unsigned)((num + d - 1) / d);
  f.sh = l - 1;
  return f;
}
__device__ __forceinline__ unsigned fast_div(unsigned n, FastDiv f) {
  return f.m ? (__umulhi(n, f.m) >> f.sh) : n;
}

// Tickets are handed out in chunk-major order: all sequences and column tiles of chunk 0, then
// chunk 1, ... (REV: the chunks from last to first), so a tile's predecessor always has a smaller
// ticket.  Within a chunk: batch element, head, column tile.  TileOrder holds the reciprocals that
// turn a ticket into its tile without divisions.
struct TileOrder {
  unsigned cols;    // tiles per chunk: sequences * column tiles
  unsigned C;       // chunks
  unsigned ntiles, nh;
  FastDiv dcols, dnt, dnh;
};
inline TileOrder tile_order_make(unsigned B, unsigned nh, unsigned C, unsigned ntiles) {
  TileOrder o;
  o.cols = B * nh * ntiles, o.C = C, o.ntiles = ntiles, o.nh = nh;
  o.dcols = fast_div_make(o.cols), o.dnt = fast_div_make(ntiles), o.dnh = fast_div_make(nh);
  return o;
}

struct ChainTile {
  int c, ctile, limit, col0, n, b, h, chunk_id, col_id;  // col_id = n * ntiles + ctile
};

// Ticket -> tile.  All quantities fit 32 bits (the host checks N * C * ntiles < 2^31).
template <bool REV, int BN>
__device__ __forceinline__ ChainTile chain_decode(int ticket, const TileOrder& o, int L) {
  ChainTile t;
  const unsigned cc = fast_div((unsigned)ticket, o.dcols);
  t.c = REV ? (int)o.C - 1 - (int)cc : (int)cc;
  t.col_id = ticket - (int)(cc * o.cols);
  t.n = (int)fast_div((unsigned)t.col_id, o.dnt);
  t.ctile = t.col_id - t.n * (int)o.ntiles;
  t.b = (int)fast_div((unsigned)t.n, o.dnh);
  t.h = t.n - t.b * (int)o.nh;
  t.chunk_id = t.n * (int)o.C + t.c;
  t.limit = min(kTileRows, L - t.c * kTileRows);
  t.col0 = t.ctile * BN;
  return t;
}

// Look-back of one column, in two parts so that other work can sit between the first request and
// its use.  words: the status words of this column, words[j * BN] that of tile j; decw[j]: the
// total decay of tile j of this sequence.  The walk starts at the neighbour of tile c (c - 1
// forward, c + 1 reverse) and ends at the first PREFIX; the first tile of a scan always
// publishes one, so the walk stays inside [0, C).  Polls are not free (every one is a trip to
// device-coherent memory), so only what is needed is requested: the neighbour's word first; a
// tile's decay only once its word shows an aggregate, together with the word of the tile beyond.
template <bool REV, int BN>
struct ChainLook {
  u64 w;  // first look at the neighbour's word
  int j;

  __device__ __forceinline__ void begin(const u64* words, int c) {
    j = REV ? c + 1 : c - 1;
    w = chain_peek(words + (int64_t)j * BN);
  }
  __device__ __forceinline__ float finish(const u64* words, const u64* decw, int C, const ChainCtl& ctl) {
    float carry = 0.f, scale = 1.f;
    for (;;) {
      const u64 sw = chain_wait(words + (int64_t)j * BN, w, ctl);
      carry = fmaf(scale, chain_value(sw), carry);
      if (chain_state(sw, ctl.epoch) == kStatePrefix) return carry;
      const int jn = REV ? j + 1 : j - 1;
      if (REV ? jn >= C : jn < 0) return carry;
      const u64 d = chain_peek(decw + j);
      w = chain_peek(words + (int64_t)jn * BN);
      scale *= chain_value(chain_wait(decw + j, d, ctl));
      j = jn;
    }
  }
};

}  // namespace ema
