// C ABI of libema_hip.so: argument validation and kernel launches.  Declarations and the
// reference launcher each entry point replaces are in include/ema_hip.h.
#include "../../include/ema_hip.h"

#include <hip/hip_runtime.h>

#include <mutex>

#include "ema_device.h"
#include "ema_gemm_kernels.h"
#include "ema_stream_kernels.h"
#include "ema_walk_kernels.h"
#include "ema_chain_kernels.h"
#include "ema_tile_kernels.h"
#include "ema_flat_kernels.h"

using namespace ema;

namespace {

struct Dims {
  int64_t batch, nh, L, T, Q, N, C;
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int elem_size(int dtype) { return dtype == EMA_BF16 ? 2 : 4; }

// Shape checks shared by every entry point that sees the sequence axis.
int check_dims(int64_t batch, int64_t nh, int64_t L, int64_t T, int64_t Q, bool has_T, Dims* d) {
  if (batch <= 0 || nh <= 0 || L <= 0 || Q <= 0 || (has_T && T <= 0)) return EMA_ERR_SHAPE;
  if (Q > EMA_MAX_CHUNK) return EMA_ERR_SHAPE;
  if (batch > (1 << 24) || nh > (1 << 16) || L > (int64_t)1 << 30 || T > (1 << 24))
    return EMA_ERR_SHAPE;
  d->batch = batch;
  d->nh = nh;
  d->L = L;
  d->T = T;
  d->Q = Q;
  d->N = batch * nh;
  d->C = (L + Q - 1) / Q;
  if (d->N * d->C > ((int64_t)1 << 30)) return EMA_ERR_SHAPE;
  return EMA_OK;
}

int check_dtype(int dtype) { return (dtype == EMA_F32 || dtype == EMA_BF16) ? EMA_OK : EMA_ERR_DTYPE; }

// A sequence tensor must allow 16-byte loads of every row segment.
int check_seq(const void* p, int64_t sb, int64_t sl, int64_t sh, int dtype, int64_t T) {
  if (!p) return EMA_ERR_NULL;
  const int epl = 16 / elem_size(dtype);
  if (T % epl || sb % epl || sl % epl || sh % epl) return EMA_ERR_ALIGN;
  if (reinterpret_cast<uintptr_t>(p) % 16) return EMA_ERR_ALIGN;
  return EMA_OK;
}

int check_f32(const void* p) {
  if (!p) return EMA_ERR_NULL;
  return reinterpret_cast<uintptr_t>(p) % 16 ? EMA_ERR_ALIGN : EMA_OK;
}

inline int launched() { return hipGetLastError() == hipSuccess ? EMA_OK : EMA_ERR_LAUNCH; }

#define EMA_TRY(expr)            \
  do {                           \
    int _s = (expr);             \
    if (_s != EMA_OK) return _s; \
  } while (0)

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---------------------------------------------------------------- launch helpers

// prob = 1: the input holds probabilities p and the sums are of log(1 - p).
int launch_cumsum(const float* A, SeqStrides sa, float* cs, const Dims& d, hipStream_t st, int prob = 0) {
  const int64_t total = d.N * d.C;
  const unsigned grid = (unsigned)((total + 3) / 4);
  hipLaunchKernelGGL(cumsum_kernel, dim3(grid), dim3(256), 0, st, A, sa, cs, (int)d.nh, (int)d.L,
                     (int)d.Q, (int)d.C, total, prob);
  return launched();
}

template <int MODE>
int launch_chunk_reduce(const void* x, SeqStrides sx, int dtype, const float* cs, float* out,
                        const Dims& d, hipStream_t st) {
  const int epl = 16 / elem_size(dtype);
  const int64_t vecs = d.T / epl;
  int cg_log2 = 0;
  while ((1 << cg_log2) < vecs && cg_log2 < 6) ++cg_log2;
  const int cg = 1 << cg_log2;
  const int ntiles = (int)((vecs + cg - 1) / cg);
  const int64_t grid = d.N * d.C * ntiles;
  if (grid > 0x7fffffff) return EMA_ERR_SHAPE;
  if (dtype == EMA_BF16)
    hipLaunchKernelGGL((chunk_reduce_kernel<bf16_t, MODE>), dim3((unsigned)grid), dim3(256), 0, st,
                       (const bf16_t*)x, sx, cs, out, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q,
                       (int)d.C, cg_log2, ntiles);
  else
    hipLaunchKernelGGL((chunk_reduce_kernel<float, MODE>), dim3((unsigned)grid), dim3(256), 0, st,
                       (const float*)x, sx, cs, out, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q,
                       (int)d.C, cg_log2, ntiles);
  return launched();
}

int launch_state_passing_fwd(const float* states, const float* cs_last, int64_t cl_sn,
                             int64_t cl_sc, float* prev, float* fin, int64_t N, int64_t C,
                             int64_t T, hipStream_t st) {
  const int tiles = (int)((T + 255) / 256);
  hipLaunchKernelGGL(state_passing_fwd_kernel, dim3((unsigned)(N * tiles)), dim3(256), 0, st,
                     states, cs_last, cl_sn, cl_sc, prev, fin, (int)C, (int)T, tiles);
  return launched();
}

int launch_state_passing_bwd(const float* prev, const float* cs_last, int64_t cl_sn,
                             int64_t cl_sc, const float* ds, float* g, float* ddA_chunk,
                             float* part, int64_t N, int64_t C, int64_t T, hipStream_t st) {
  const int tiles = (int)((T + 255) / 256);
  const int nw = (int)((T + 63) / 64);
  if (!ddA_chunk) {  // only the recurrence; no <prev, g> products
    hipLaunchKernelGGL(state_passing_bwd_kernel<false>, dim3((unsigned)(N * tiles)), dim3(256), 0,
                       st, prev, cs_last, cl_sn, cl_sc, ds, g, part, (int)C, (int)T, tiles, nw);
    return launched();
  }
  hipLaunchKernelGGL(state_passing_bwd_kernel<true>, dim3((unsigned)(N * tiles)), dim3(256), 0, st,
                     prev, cs_last, cl_sn, cl_sc, ds, g, part, (int)C, (int)T, tiles, nw);
  EMA_TRY(launched());
  const int64_t total = N * C;
  hipLaunchKernelGGL(state_passing_bwd_finish_kernel, dim3((unsigned)((total + 255) / 256)),
                     dim3(256), 0, st, part, cs_last, cl_sn, cl_sc, ddA_chunk, (int)C, nw, total);
  return launched();
}

// Kernels that ask for more dynamic LDS than the default limit must opt in once.
template <typename K>
int allow_smem(K kernel, int bytes) {
  if (bytes <= 48 * 1024) return EMA_OK;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess
             ? EMA_OK
             : EMA_ERR_LAUNCH;
}

constexpr int kWalkBnBf16 = 128;  // column tile of the per-stage intra-chunk kernels, bf16
constexpr int kWalkBnF32 = 64;    // and f32 (both are 256 bytes per row)

template <typename T, int BN, bool REVERSE>
int launch_chunk_scan_t(const void* in, SeqStrides si, const float* cs, const float* vec, void* out,
                        SeqStrides so, const Dims& d, hipStream_t st) {
  const int ntiles = (int)((d.T + BN - 1) / BN);
  const int64_t grid = d.N * d.C * ntiles;
  if (grid > 0x7fffffff) return EMA_ERR_SHAPE;
  const int smem = WalkCfg<T, BN>::smem_bytes(1, 1);
  auto kernel = chunk_scan_walk_kernel<T, BN, REVERSE>;
  EMA_TRY(allow_smem(kernel, smem));
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), smem, st, (const T*)in, si, cs, vec,
                     (T*)out, so, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q, (int)d.C, ntiles);
  return launched();
}

template <bool REVERSE>
int launch_chunk_gemm(const void* in, SeqStrides si, int dtype, const float* cs, const float* vec,
                      void* out, SeqStrides so, const Dims& d, hipStream_t st) {
  if (dtype == EMA_BF16)
    return launch_chunk_scan_t<bf16_t, kWalkBnBf16, REVERSE>(in, si, cs, vec, out, so, d, st);
  return launch_chunk_scan_t<float, kWalkBnF32, REVERSE>(in, si, cs, vec, out, so, d, st);
}

template <int MODE>
int launch_row_dot(const void* x, SeqStrides sx, int dtype, const float* vec, const float* cs,
                   float* out, int raw, const Dims& d, hipStream_t st) {
  const unsigned grid = (unsigned)(d.N * d.C);
  if (dtype == EMA_BF16)
    hipLaunchKernelGGL((row_dot_kernel<bf16_t, MODE>), dim3(grid), dim3(kRowDotThreads), 0, st,
                       (const bf16_t*)x, sx, vec, cs, out, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q,
                       (int)d.C, raw);
  else
    hipLaunchKernelGGL((row_dot_kernel<float, MODE>), dim3(grid), dim3(kRowDotThreads), 0, st, (const float*)x,
                       sx, vec, cs, out, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q, (int)d.C, raw);
  return launched();
}

// The backward chunks the sequence by 128 internally, whatever the chunk size of the
// interface: internal_dims describes that chunking.
Dims internal_dims(const Dims& d) {
  Dims di = d;
  di.Q = kTileRows;
  di.C = (d.L + kTileRows - 1) / kTileRows;
  return di;
}

int bwd_col_tiles(const Dims& d, int dtype) {
  const int bn = dtype == EMA_BF16 ? kWalkBnBf16 : kWalkBnF32;
  return (int)((d.T + bn - 1) / bn);
}

// ---------------------------------------------------------------- chained single-pass kernels

// Records an optional hipEvent_t (NULL = nothing) on the launch stream.
inline int record_event(void* ev, hipStream_t st) {
  if (!ev) return EMA_OK;
  return hipEventRecord(reinterpret_cast<hipEvent_t>(ev), st) == hipSuccess ? EMA_OK : EMA_ERR_LAUNCH;
}

// Launches a kernel that uses no dynamic LDS, with optional events (hipEvent_t, either may be NULL)
// recorded on the stream right before and right after it.  In a sequence of launches the interval
// between them is the kernel's share of the stream's time: it starts when the work before is
// complete (written back), which is also how a kernel trace accounts a dispatch; the runtime's own
// start / stop stamps of the dispatch leave out what the hand-over between two kernels costs.
template <typename... Args>
int launch_timed(void (*kernel)(Args...), dim3 grid, dim3 block, hipStream_t st, void* ev0, void* ev1,
                 Args... args) {
  if (ev0 && hipEventRecord(reinterpret_cast<hipEvent_t>(ev0), st) != hipSuccess) return EMA_ERR_LAUNCH;
  hipLaunchKernelGGL(kernel, grid, block, 0, st, args...);
  if (ev1 && hipEventRecord(reinterpret_cast<hipEvent_t>(ev1), st) != hipSuccess) return EMA_ERR_LAUNCH;
  return EMA_OK;
}

// Workgroups of a persistent kernel that can be resident at once on the current device.
#ifndef EMA_MAX_WGS_PER_CU  // development knob: cap on the resident workgroups per compute unit
#define EMA_MAX_WGS_PER_CU 64
#endif
template <typename K>
int resident_blocks(K kernel, int threads, int smem) {
  int dev = 0, ncu = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) ncu = 256;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel),
                                                   threads, smem) != hipSuccess || per_cu < 1)
    per_cu = 1;
  if (per_cu > EMA_MAX_WGS_PER_CU) per_cu = EMA_MAX_WGS_PER_CU;
  return ncu * per_cu;
}

inline int64_t padded_dim(int64_t T) { return (T + 255) / 256 * 256; }

// Workspace of one chained kernel: the header, one total-decay word per (sequence, tile) and one
// status word per (sequence, tile, column).  The header sits at the start of the buffer whatever
// the shape, so that a buffer can serve calls of different shapes one after the other.
struct ChainWs {
  ChainHeader* hdr;
  u64* decw;
  u64* status;
};
inline size_t chain_decw_bytes(const Dims& di) { return align_up((size_t)(di.N * di.C) * sizeof(u64), 256); }
inline size_t chain_status_bytes(const Dims& di) {
  return align_up((size_t)(di.N * di.C * padded_dim(di.T)) * sizeof(u64), 256);
}
inline size_t chain_ws_bytes(const Dims& di) {
  return sizeof(ChainHeader) + chain_decw_bytes(di) + chain_status_bytes(di);
}
inline ChainWs chain_carve(void* base, const Dims& di) {
  ChainWs w;
  char* p = static_cast<char*>(base);
  w.hdr = reinterpret_cast<ChainHeader*>(p);
  w.decw = reinterpret_cast<u64*>(p + sizeof(ChainHeader));
  w.status = reinterpret_cast<u64*>(p + sizeof(ChainHeader) + chain_decw_bytes(di));
  return w;
}

// Zero fill with a kernel (a memset node in a captured graph is not wanted here).
int launch_clear(void* base, size_t bytes, hipStream_t st) {
  const int64_t n16 = (int64_t)((bytes + 15) / 16);
  if (n16 == 0) return EMA_OK;
  if ((n16 + 255) / 256 > 0x7fffffff) return EMA_ERR_SHAPE;
  hipLaunchKernelGGL(chain_clear_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, st,
                     static_cast<uint4*>(base), n16);
  return launched();
}

// Shape of the register-tile single-pass kernels: columns per lane (a tile is 128 rows by
// 64 times that many columns), rows per lane (128 / RPL waves per workgroup), waves per SIMD
// the register allocation must allow.
#ifndef EMA_FWD_SHAPE  // columns per lane, rows per lane, waves per SIMD
#define EMA_FWD_SHAPE 4, 8, 4
#endif
#ifndef EMA_BWD_SHAPE
#define EMA_BWD_SHAPE 4, 8, 4
#endif
struct TileShape {
  int cpl, rpl, minw;
};
struct TileBf16 {
  static constexpr TileShape F{EMA_FWD_SHAPE}, B{EMA_BWD_SHAPE};
  static constexpr int FWD_CPL = F.cpl, FWD_RPL = F.rpl, FWD_MINW = F.minw;
  static constexpr int BWD_CPL = B.cpl, BWD_RPL = B.rpl, BWD_MINW = B.minw;
};
struct TileF32 {
  static constexpr int FWD_CPL = 2, FWD_RPL = 8, FWD_MINW = 4;
  static constexpr int BWD_CPL = 2, BWD_RPL = 8, BWD_MINW = 4;
};

inline TileOrder make_order(const Dims& di, int ntiles) {
  return tile_order_make((unsigned)di.batch, (unsigned)di.nh, (unsigned)di.C, (unsigned)ntiles);
}

// ready: the chained part of the workspace is as a zero fill or an earlier call left it;
// otherwise it is cleared first.
template <typename T, typename S, bool XP>
int launch_fwd_tile_t(const void* x, SeqStrides sx, const float* A, SeqStrides sa, void* y, SeqStrides sy,
                      float* prev128, float* prev_coarse, int ratio, float* fin, const float* init,
                      void* chain_base, bool ready, const Dims& di, hipStream_t st, void* ev0, void* ev1) {
  using Cfg = TileCfg<T, S::FWD_CPL, S::FWD_RPL>;
  constexpr int BN = Cfg::BN, NT = Cfg::NT;
  const int ntiles = (int)((di.T + BN - 1) / BN);
  const int64_t cols = di.N * ntiles, total = cols * di.C;
  if (total > 0x7fffffff) return EMA_ERR_SHAPE;
  if (!ready) EMA_TRY(launch_clear(chain_base, chain_ws_bytes(di), st));
  const ChainWs w = chain_carve(chain_base, di);
  auto kernel = fwd_tile_kernel<T, S::FWD_CPL, S::FWD_RPL, S::FWD_MINW, XP>;
  const int64_t cap = resident_blocks(kernel, NT, 0);
  EMA_TRY(launch_timed(kernel, dim3((unsigned)(total < cap ? total : cap)), dim3(NT), st, ev0, ev1, (const T*)x,
                       sx, A, sa, (T*)y, sy, prev128, prev_coarse, ratio, fin, init, w.hdr, w.decw, w.status,
                       (int)di.nh, (int)di.L, (int)di.T, (int)di.C, ntiles, (int)cols, (int)total,
                       make_order(di, ntiles)));
  return launched();
}

template <typename T, typename S, bool WRITE_Y, bool XP>
int launch_bwd_tile_k(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* A,
                      SeqStrides sa, const float* prev128, void* dx, SeqStrides sdx, void* y, SeqStrides sy,
                      float* part, const float* dfinal, float* dinit, void* chain_base, bool ready,
                      const Dims& di, hipStream_t st, void* ev0, void* ev1) {
  using Cfg = TileCfg<T, S::BWD_CPL, S::BWD_RPL>;
  constexpr int BN = Cfg::BN, NT = Cfg::NT;
  const int ntiles = (int)((di.T + BN - 1) / BN);
  const int64_t cols = di.N * ntiles, total = cols * di.C;
  if (total > 0x7fffffff) return EMA_ERR_SHAPE;
  if (!ready) EMA_TRY(launch_clear(chain_base, chain_ws_bytes(di), st));
  const ChainWs w = chain_carve(chain_base, di);
  auto kernel = bwd_tile_kernel<T, S::BWD_CPL, S::BWD_RPL, S::BWD_MINW, WRITE_Y, XP>;
  const int64_t cap = resident_blocks(kernel, NT, 0);
  EMA_TRY(launch_timed(kernel, dim3((unsigned)(total < cap ? total : cap)), dim3(NT), st, ev0, ev1, (const T*)x,
                       sx, (const T*)dy, sd, A, sa, prev128, (T*)dx, sdx, (T*)y, sy, part, dfinal, dinit, w.hdr,
                       w.decw, w.status, (int)di.nh, (int)di.L, (int)di.T, (int)di.C, ntiles, (int)cols,
                       (int)total, make_order(di, ntiles), (const float*)nullptr));
  return launched();
}

template <typename T, typename S, bool XP>
int launch_bwd_tile_t(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* A,
                      SeqStrides sa, const float* prev128, void* dx, SeqStrides sdx, void* y, SeqStrides sy,
                      float* part, const float* dfinal, float* dinit, void* chain_base, bool ready,
                      const Dims& di, hipStream_t st, void* ev0, void* ev1) {
  if (y)
    return launch_bwd_tile_k<T, S, true, XP>(x, sx, dy, sd, A, sa, prev128, dx, sdx, y, sy, part, dfinal, dinit,
                                             chain_base, ready, di, st, ev0, ev1);
  return launch_bwd_tile_k<T, S, false, XP>(x, sx, dy, sd, A, sa, prev128, dx, sdx, nullptr, sy, part, dfinal,
                                            dinit, chain_base, ready, di, st, ev0, ev1);
}

template <typename S>
constexpr int tile_parts_per_dim(int64_t T) {
  return (int)((T + 64 * S::BWD_CPL - 1) / (64 * S::BWD_CPL));
}

// dx, optionally the recomputed y, and the log-decay gradient in one pass over x and dy, with the
// states entering every 128-row chunk from both sides given (prev, g): the backward single-pass
// kernel with nothing to chain.  di is the 128-row chunking the kernel works on (cs, prev, g follow
// it); d fixes the (N, C, Q) layout of ddA.
template <typename T, typename S>
int launch_bwd_tile_given(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* cs,
                          const float* prev, const float* g, void* dx, SeqStrides sdx, void* y, SeqStrides sy,
                          float* part, const Dims& di, hipStream_t st) {
  using Cfg = TileCfg<T, S::BWD_CPL, S::BWD_RPL>;
  constexpr int BN = Cfg::BN, NT = Cfg::NT;
  const int ntiles = (int)((di.T + BN - 1) / BN);
  const int64_t cols = di.N * ntiles, total = cols * di.C;
  if (total > 0x7fffffff) return EMA_ERR_SHAPE;
  const SeqStrides sa{di.nh * di.C * kTileRows, 1, di.C * kTileRows};  // cs is dense (N, C, 128)
  auto launch = [&](auto kernel) {
    const int64_t cap = resident_blocks(kernel, NT, 0);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(total < cap ? total : cap)), dim3(NT), 0, st, (const T*)x, sx,
                       (const T*)dy, sd, cs, sa, prev, (T*)dx, sdx, (T*)y, sy, part, (const float*)nullptr,
                       (float*)nullptr, (ChainHeader*)nullptr, (u64*)nullptr, (u64*)nullptr, (int)di.nh, (int)di.L,
                       (int)di.T, (int)di.C, ntiles, (int)cols, (int)total, make_order(di, ntiles), g);
  };
  if (y) launch(bwd_tile_kernel<T, S::BWD_CPL, S::BWD_RPL, S::BWD_MINW, true, false, true>);
  else launch(bwd_tile_kernel<T, S::BWD_CPL, S::BWD_RPL, S::BWD_MINW, false, false, true>);
  return launched();
}

int run_bwd_fused(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, int dtype,
                  const float* cs, const float* prev, const float* g, void* dx, SeqStrides sdx,
                  void* y, SeqStrides sy, float* ddA, float* part, const Dims& d, const Dims& di,
                  hipStream_t st) {
  int parts;
  if (dtype == EMA_BF16) {
    EMA_TRY((launch_bwd_tile_given<bf16_t, TileBf16>(x, sx, dy, sd, cs, prev, g, dx, sdx, y, sy, part, di, st)));
    parts = tile_parts_per_dim<TileBf16>(di.T);
  } else {
    EMA_TRY((launch_bwd_tile_given<float, TileF32>(x, sx, dy, sd, cs, prev, g, dx, sdx, y, sy, part, di, st)));
    parts = tile_parts_per_dim<TileF32>(di.T);
  }
  const int64_t total = d.N * d.C * d.Q;
  hipLaunchKernelGGL(dA_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, part,
                     ddA, (int)d.L, (int)d.Q, (int)d.C, (int)di.C, parts, total);
  return launched();
}

// Workspace of B6: column sums per row tile and row sums of the kernel that forms the product, then
// the per-column-tile dots of the factored form and one flag per chunk.
struct DaWs {
  float *part, *rowsum, *flat;
  int* steep;
  size_t bytes;
};
// Columns per workgroup of the factored form: the single-pass kernels' tile; for float32 chunks of
// three or four 128-row sub-tiles half of it (a chunk's x rows stay in registers, and eight bytes per
// row and lane are too many there).
template <typename T>
constexpr int kFlatLongDiv = sizeof(T) == 4 ? 2 : 1;
inline int da_flat_cols(const Dims& d, int dtype) {
  const int wide = dtype == EMA_BF16 ? 64 * TileBf16::BWD_CPL : 64 * TileF32::BWD_CPL;
  const int div = dtype == EMA_BF16 ? kFlatLongDiv<bf16_t> : kFlatLongDiv<float>;
  return d.Q > 2 * kTileRows && d.Q <= 4 * kTileRows ? wide / div : wide;
}
inline int da_flat_tiles(const Dims& d, int dtype) {
  const int bn = da_flat_cols(d, dtype);
  return (int)((d.T + bn - 1) / bn);
}
// The factored form takes every chunk size the library does: up to four 128-row sub-tiles with the
// chunk's x rows kept in registers, more with x read twice.
constexpr int kFlatMaxChunk = EMA_MAX_CHUNK;
constexpr int kFlatMaxKept = 4 * kTileRows;
DaWs carve_da(void* base, const Dims& d, int dtype) {
  DaWs w;
  size_t off = 0;
  char* p = static_cast<char*>(base);
  auto take = [&](size_t bytes) {
    char* r = p + off;
    off += align_up(bytes, 256);
    return r;
  };
  const int64_t MT = (d.Q + kBM - 1) / kBM;
  w.part = reinterpret_cast<float*>(take((size_t)(d.N * d.C * MT * d.Q) * sizeof(float)));
  w.rowsum = reinterpret_cast<float*>(take((size_t)(d.N * d.C * d.Q) * sizeof(float)));
  const bool flat = d.Q <= kFlatMaxChunk;
  w.flat = reinterpret_cast<float*>(take(flat ? (size_t)(d.N * d.C * d.Q) * da_flat_tiles(d, dtype) * sizeof(float) : 0));
  w.steep = reinterpret_cast<int*>(take(flat ? (size_t)(d.N * d.C) * sizeof(int) : 0));
  w.bytes = off;
  return w;
}

template <typename T, int CPL, int RPL, int KT>
int launch_da_flat_k(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* cs,
                     const DaWs& w, const Dims& d, hipStream_t st) {
  using Cfg = TileCfg<T, CPL, RPL>;
  constexpr int smem = FlatCfg<T, CPL, RPL, KT>::smem_bytes;
  const int ntiles = (int)((d.T + Cfg::BN - 1) / Cfg::BN);
  const int64_t total = d.N * d.C * ntiles;
  if (total > 0x7fffffff) return EMA_ERR_SHAPE;
  auto kernel = da_flat_kernel<T, CPL, RPL, KT>;
  EMA_TRY(allow_smem(kernel, smem));
  const int64_t cap = resident_blocks(kernel, Cfg::NT, smem);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(total < cap ? total : cap)), dim3(Cfg::NT), smem, st, (const T*)x, sx,
                     (const T*)dy, sd, cs, w.flat, w.steep, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q, (int)d.C,
                     ntiles, (int)total);
  return launched();
}
template <typename T, int CPL, int RPL>
int launch_da_flat_long(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* cs,
                        const DaWs& w, const Dims& d, hipStream_t st) {
  using Cfg = TileCfg<T, CPL, RPL>;
  constexpr int smem = FlatLongCfg<T, CPL, RPL>::smem_bytes;
  const int ntiles = (int)((d.T + Cfg::BN - 1) / Cfg::BN);
  const int64_t total = d.N * d.C * ntiles;
  if (total > 0x7fffffff) return EMA_ERR_SHAPE;
  auto kernel = da_flat_long_kernel<T, CPL, RPL>;
  EMA_TRY(allow_smem(kernel, smem));
  const int64_t cap = resident_blocks(kernel, Cfg::NT, smem);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(total < cap ? total : cap)), dim3(Cfg::NT), smem, st, (const T*)x, sx,
                     (const T*)dy, sd, cs, w.flat, w.steep, (int)d.nh, (int)d.L, (int)d.T, (int)d.Q, (int)d.C,
                     ntiles, (int)total);
  return launched();
}
template <typename T, typename S>
int launch_da_flat(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, const float* cs,
                   const DaWs& w, const Dims& d, hipStream_t st) {
  constexpr int CPL = S::BWD_CPL, RPL = S::BWD_RPL;
  if (d.Q > kFlatMaxKept) return launch_da_flat_long<T, CPL, RPL>(x, sx, dy, sd, cs, w, d, st);
  static_assert(CPL % kFlatLongDiv<T> == 0, "long chunks take a part of the columns");
  switch ((d.Q + kTileRows - 1) / kTileRows) {
    case 1: return launch_da_flat_k<T, CPL, RPL, 1>(x, sx, dy, sd, cs, w, d, st);
    case 2: return launch_da_flat_k<T, CPL, RPL, 2>(x, sx, dy, sd, cs, w, d, st);
    case 3: return launch_da_flat_k<T, CPL / kFlatLongDiv<T>, RPL, 3>(x, sx, dy, sd, cs, w, d, st);
    default: return launch_da_flat_k<T, CPL / kFlatLongDiv<T>, RPL, 4>(x, sx, dy, sd, cs, w, d, st);
  }
}

// B6.  Every chunk goes through the factored form first; the kernel that forms the product and its
// finish then take the chunks in which the cumsum rises somewhere (none, for decays) and the finish
// of the factored form the others.
int launch_da(const void* x, SeqStrides sx, const void* dy, SeqStrides sd, int dtype,
              const float* cs, float* ddA_intra, const DaWs& w, const Dims& d, hipStream_t st) {
  const int MT = (int)((d.Q + kBM - 1) / kBM);
  const int64_t grid = d.N * d.C * MT;
  if (grid > 0x7fffffff) return EMA_ERR_SHAPE;
  // the factored form reads a chunk's rows at 32-bit byte offsets from the chunk's first row and
  // tells rows apart by their offset: rows must not overlap and a chunk must span less than 2 GiB
  auto fits = [&](const SeqStrides& s) {
    return s.sl >= d.T && (d.Q * s.sl + 256) * (int64_t)elem_size(dtype) < (int64_t)0x7fffffff;
  };
  const bool flat = d.Q <= kFlatMaxChunk && fits(sx) && fits(sd);
  if (flat) {
    if (dtype == EMA_BF16) EMA_TRY((launch_da_flat<bf16_t, TileBf16>(x, sx, dy, sd, cs, w, d, st)));
    else EMA_TRY((launch_da_flat<float, TileF32>(x, sx, dy, sd, cs, w, d, st)));
  }
  const int* only = flat ? w.steep : nullptr;
  if (dtype == EMA_BF16)
    hipLaunchKernelGGL((da_gemm_kernel<bf16_t>), dim3((unsigned)grid), dim3(256), 0, st,
                       (const bf16_t*)x, sx, (const bf16_t*)dy, sd, cs, w.part, w.rowsum, (int)d.nh,
                       (int)d.L, (int)d.T, (int)d.Q, (int)d.C, MT, nullptr, nullptr, 1, 1, only);
  else
    hipLaunchKernelGGL((da_gemm_kernel<float>), dim3((unsigned)grid), dim3(256), 0, st,
                       (const float*)x, sx, (const float*)dy, sd, cs, w.part, w.rowsum, (int)d.nh,
                       (int)d.L, (int)d.T, (int)d.Q, (int)d.C, MT, nullptr, nullptr, 1, 1, only);
  EMA_TRY(launched());
  const int64_t total = d.N * d.C;
  hipLaunchKernelGGL(da_finish_kernel<kBM>, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, st, w.part,
                     w.rowsum, ddA_intra, (int)d.Q, MT, total, only);
  if (flat) {
    EMA_TRY(launched());
    const int64_t n = total * d.Q;
    hipLaunchKernelGGL(da_flat_finish_kernel<256>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, w.flat, w.steep,
                       ddA_intra, (int)d.Q, da_flat_tiles(d, dtype), n);
  }
  return launched();
}

// Workspace of the sequence-level entry points: the chained part first, then (backward) the
// dA partials.
struct SeqWs {
  void* chain;
  float* part;
  size_t bytes;
};
SeqWs carve_seq(void* base, const Dims& di, bool backward) {
  SeqWs w;
  char* p = static_cast<char*>(base);
  size_t off = chain_ws_bytes(di);
  w.chain = base;
  w.part = nullptr;
  if (backward) {
    const int pb = tile_parts_per_dim<TileBf16>(di.T), pf = tile_parts_per_dim<TileF32>(di.T);
    w.part = reinterpret_cast<float*>(p + off);
    off += align_up((size_t)(di.N * di.C * di.Q) * (size_t)(pb > pf ? pb : pf) * sizeof(float), 256);
  }
  w.bytes = off;
  return w;
}

// ---------------------------------------------------------------- file-scope scratch
// Workspace of ema_seq_fwd_static: one copy per GPU that loads the library, held until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// address the kernels get is looked up once per device and kept.
constexpr size_t kScratchBytes = EMA_STATIC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device.
int scratch_address(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return EMA_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return EMA_ERR_LAUNCH;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return EMA_OK;
}

}  // namespace

// ====================================================================================

extern "C" {

const char* ema_version(void) { return "ema_hip 0.1 (gfx950)"; }

const char* ema_status_string(int status) {
  switch (status) {
    case EMA_OK: return "ok";
    case EMA_ERR_NULL: return "null pointer";
    case EMA_ERR_SHAPE: return "bad shape";
    case EMA_ERR_ALIGN: return "dim, stride or pointer not 16-byte aligned";
    case EMA_ERR_DTYPE: return "unknown dtype";
    case EMA_ERR_UNSUPPORTED: return "unsupported";
    case EMA_ERR_LAUNCH: return "kernel launch failed";
    case EMA_ERR_TOO_LARGE: return "problem exceeds the fixed scratch of the allocation-free entry point";
    default: return "unknown status";
  }
}

int ema_chunk_cumsum_fwd(const float* A, int64_t a_sb, int64_t a_sl, int64_t a_sh, float* cs,
                         int64_t batch, int64_t nheads, int64_t seqlen, int64_t chunk,
                         void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, 1, chunk, false, &d));
  if (!A || !cs) return EMA_ERR_NULL;
  return launch_cumsum(A, SeqStrides{a_sb, a_sl, a_sh}, cs, d, as_stream(stream));
}

int ema_chunk_state_fwd(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                        const float* cs, float* states, int64_t batch, int64_t nheads,
                        int64_t seqlen, int64_t dim, int64_t chunk, void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  if (!cs || !states) return EMA_ERR_NULL;
  return launch_chunk_reduce<0>(x, SeqStrides{x_sb, x_sl, x_sh}, dtype, cs, states, d,
                                as_stream(stream));
}

int ema_state_passing_fwd(const float* states, const float* cs_last, int64_t cl_sn, int64_t cl_sc,
                          float* prev, float* final_state, int64_t nseq, int64_t nchunks,
                          int64_t dim, void* stream) {
  if (nseq <= 0 || nchunks <= 0 || dim <= 0) return EMA_ERR_SHAPE;
  if (nseq * ((dim + 255) / 256) > 0x7fffffff) return EMA_ERR_SHAPE;
  if (!states || !cs_last || !prev || !final_state) return EMA_ERR_NULL;
  return launch_state_passing_fwd(states, cs_last, cl_sn, cl_sc, prev, final_state, nseq, nchunks,
                                  dim, as_stream(stream));
}

int ema_scan_fwd(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                 const float* cs, const float* prev, void* y, int64_t y_sb, int64_t y_sl,
                 int64_t y_sh, int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                 int64_t chunk, void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(y, y_sb, y_sl, y_sh, dtype, dim));
  if (!cs || !prev) return EMA_ERR_NULL;
  return launch_chunk_gemm<false>(x, SeqStrides{x_sb, x_sl, x_sh}, dtype, cs, prev, y,
                                  SeqStrides{y_sb, y_sl, y_sh}, d, as_stream(stream));
}

// Workspace of ema_fwd: the chained part first (left alone by the staged path, so that the
// buffer stays ready for the single-pass kernels), then room for the 128-row chunk-entry states
// when the caller keeps none, or for the chunk states of the staged path.
struct FwdWs {
  void* chain;
  float* scratch;
  size_t bytes;
};
static FwdWs carve_fwd(void* base, const Dims& d) {
  const Dims di = internal_dims(d);
  FwdWs w;
  char* p = static_cast<char*>(base);
  size_t off = chain_ws_bytes(di);
  w.chain = base;
  w.scratch = reinterpret_cast<float*>(p + off);
  const size_t n128 = (size_t)(di.N * di.C * di.T), nq = (size_t)(d.N * d.C * d.T);
  off += align_up((n128 > nq ? n128 : nq) * sizeof(float), 256);
  w.bytes = off;
  return w;
}

size_t ema_fwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                               int64_t chunk) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, chunk, true, &d) != EMA_OK) return 0;
  return carve_fwd(nullptr, d).bytes;
}

int ema_stream_copy(const void* a, const void* b, void* dst, size_t bytes, void* stream) {
  if (!a || !dst) return EMA_ERR_NULL;
  if (bytes % 16 || reinterpret_cast<uintptr_t>(a) % 16 || reinterpret_cast<uintptr_t>(dst) % 16 ||
      reinterpret_cast<uintptr_t>(b) % 16)
    return EMA_ERR_ALIGN;
  const int64_t n16 = (int64_t)(bytes / 16);
  if (n16 == 0) return EMA_OK;
  if ((n16 + 255) / 256 > 0x7fffffff) return EMA_ERR_SHAPE;
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const uint4*>(a), static_cast<const uint4*>(b), static_cast<uint4*>(dst), n16);
  return launched();
}

int ema_tile_pattern_copy(const void* src, const void* src2, void* dst, int64_t slabs, int64_t rows, int64_t row_bytes,
                          int rowmap, void* stream) {
  if (!src || !dst) return EMA_ERR_NULL;
  if (src2 && rowmap != 0) return EMA_ERR_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(src2) % 16) return EMA_ERR_ALIGN;
  if (slabs <= 0 || rows <= 0 || row_bytes <= 0 || rows % 128 || row_bytes % 512) return EMA_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(dst) % 16) return EMA_ERR_ALIGN;
  const int64_t pieces = row_bytes / 512, tiles = slabs * (rows / 128) * pieces;
  if (tiles > 0x7fffffff || slabs > 0x7fffffff / pieces) return EMA_ERR_SHAPE;
  if (rowmap < 0 || rowmap > 3) return EMA_ERR_UNSUPPORTED;
  // one workgroup per compute unit, as the single-pass kernels run
  int dev = 0, ncu = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return EMA_ERR_LAUNCH;
  const dim3 grid((unsigned)(tiles < ncu ? tiles : ncu));
  const char* s8 = static_cast<const char*>(src);
  const char* s28 = static_cast<const char*>(src2);
  char* d8 = static_cast<char*>(dst);
  const int rb = (int)(rows / 128);
  hipStream_t st = as_stream(stream);
  if (rowmap == 0) {
    hipLaunchKernelGGL(tile_copy_shape_kernel<16>, grid, dim3(1024), 0, st, s8, s28, d8, (int)slabs, rb, (int)pieces,
                       row_bytes, rows * row_bytes);
  } else if (rowmap == 3) {
    hipLaunchKernelGGL(tile_copy_shape_kernel<8>, grid, dim3(512), 0, st, s8, (const char*)nullptr, d8, (int)slabs, rb,
                       (int)pieces, row_bytes, rows * row_bytes);
  } else if (rowmap == 1) {
    hipLaunchKernelGGL(tile_copy_kernel, grid, dim3(512), 0, st, s8, d8, (int)slabs, rb, (int)pieces, row_bytes,
                       rows * row_bytes);
  } else {
    constexpr int smem = 2 * 128 * 512;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(tile_copy_exchange_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess)
      return EMA_ERR_LAUNCH;
    hipLaunchKernelGGL(tile_copy_exchange_kernel, grid, dim3(512), smem, st, s8, d8, (int)slabs, rb, (int)pieces,
                       row_bytes, rows * row_bytes);
  }
  return launched();
}

int ema_workspace_clear(void* workspace, size_t bytes, void* stream) {
  EMA_TRY(check_f32(workspace));
  return launch_clear(workspace, bytes, as_stream(stream));
}

int ema_fwd(const float* A, int64_t a_sb, int64_t a_sl, int64_t a_sh, const void* x, int64_t x_sb,
            int64_t x_sl, int64_t x_sh, int dtype, void* y, int64_t y_sb, int64_t y_sl,
            int64_t y_sh, float* cs, float* prev, float* final_state, float* prev128,
            void* workspace, size_t workspace_bytes, int workspace_ready, int64_t batch, int64_t nheads,
            int64_t seqlen, int64_t dim, int64_t chunk, void* stream, void* ev_start, void* ev_stop) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(y, y_sb, y_sl, y_sh, dtype, dim));
  if (!A || !cs || !prev || !final_state) return EMA_ERR_NULL;
  EMA_TRY(check_f32(workspace));
  if (workspace_bytes < ema_fwd_workspace_bytes(batch, nheads, seqlen, dim, chunk))
    return EMA_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  const SeqStrides sx{x_sb, x_sl, x_sh}, sy{y_sb, y_sl, y_sh}, sa{a_sb, a_sl, a_sh};
  EMA_TRY(launch_cumsum(A, sa, cs, d, st));  // an output of this entry point; the scan below does not read it
  if (chunk % kTileRows == 0) {
    // Single pass over x: the scan is computed on 128-row chunks with the inter-chunk state
    // handed over inside the kernel; the states at the caller's chunk boundaries are every
    // (chunk/128)-th of them.
    const Dims di = internal_dims(d);
    const FwdWs w = carve_fwd(workspace, d);
    const int ratio = (int)(chunk / kTileRows);
    float* p128 = prev128 ? prev128 : (ratio == 1 ? prev : w.scratch);
    float* coarse = p128 == prev ? nullptr : prev;
    if (dtype == EMA_BF16)
      return launch_fwd_tile_t<bf16_t, TileBf16, false>(x, sx, A, sa, y, sy, p128, coarse, ratio, final_state,
                                                        nullptr, w.chain, workspace_ready != 0, di, st,
                                                        ev_start, ev_stop);
    return launch_fwd_tile_t<float, TileF32, false>(x, sx, A, sa, y, sy, p128, coarse, ratio, final_state,
                                                    nullptr, w.chain, workspace_ready != 0, di, st, ev_start,
                                                    ev_stop);
  }
  if (prev128) return EMA_ERR_UNSUPPORTED;  // only produced when chunk is a multiple of 128
  float* states = carve_fwd(workspace, d).scratch;
  EMA_TRY(record_event(ev_start, st));
  EMA_TRY(launch_chunk_reduce<0>(x, sx, dtype, cs, states, d, st));
  EMA_TRY(launch_state_passing_fwd(states, cs + (d.Q - 1), d.C * d.Q, d.Q, prev, final_state, d.N,
                                   d.C, d.T, st));
  EMA_TRY(launch_chunk_gemm<false>(x, sx, dtype, cs, prev, y, sy, d, st));
  return record_event(ev_stop, st);
}

int ema_chunk_scan_bwd_dstates(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                               int dtype, const float* cs, float* ds, int64_t batch, int64_t nheads,
                               int64_t seqlen, int64_t dim, int64_t chunk, void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  if (!cs || !ds) return EMA_ERR_NULL;
  return launch_chunk_reduce<1>(dy, SeqStrides{dy_sb, dy_sl, dy_sh}, dtype, cs, ds, d,
                                as_stream(stream));
}

size_t ema_state_passing_bwd_workspace_bytes(int64_t nseq, int64_t nchunks, int64_t dim) {
  if (nseq <= 0 || nchunks <= 0 || dim <= 0) return 0;
  return align_up((size_t)(nseq * nchunks * ((dim + 63) / 64)) * sizeof(float), 256);
}

int ema_state_passing_bwd(const float* prev, const float* cs_last, int64_t cl_sn, int64_t cl_sc,
                          const float* ds, float* g, float* ddA_chunk, void* workspace,
                          size_t workspace_bytes, int64_t nseq, int64_t nchunks, int64_t dim,
                          void* stream) {
  if (nseq <= 0 || nchunks <= 0 || dim <= 0) return EMA_ERR_SHAPE;
  if (nseq * ((dim + 255) / 256) > 0x7fffffff) return EMA_ERR_SHAPE;
  if (!prev || !cs_last || !ds || !g || !ddA_chunk || !workspace) return EMA_ERR_NULL;
  if (workspace_bytes < ema_state_passing_bwd_workspace_bytes(nseq, nchunks, dim))
    return EMA_ERR_SHAPE;
  return launch_state_passing_bwd(prev, cs_last, cl_sn, cl_sc, ds, g, ddA_chunk,
                                  static_cast<float*>(workspace), nseq, nchunks, dim,
                                  as_stream(stream));
}

int ema_chunk_scan_chunk_state_bwd_dx(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                                      int dtype, const float* cs, const float* g, void* dx,
                                      int64_t dx_sb, int64_t dx_sl, int64_t dx_sh, int64_t batch,
                                      int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk,
                                      void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  EMA_TRY(check_seq(dx, dx_sb, dx_sl, dx_sh, dtype, dim));
  if (!cs || !g) return EMA_ERR_NULL;
  return launch_chunk_gemm<true>(dy, SeqStrides{dy_sb, dy_sl, dy_sh}, dtype, cs, g, dx,
                                 SeqStrides{dx_sb, dx_sl, dx_sh}, d, as_stream(stream));
}

int ema_chunk_state_bwd_db(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                           const float* cs, const float* g, float* ddA_next, int raw, int64_t batch,
                           int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk,
                           void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  if (!cs || !ddA_next) return EMA_ERR_NULL;
  EMA_TRY(check_f32(g));
  if (dim % 4) return EMA_ERR_ALIGN;
  return launch_row_dot<0>(x, SeqStrides{x_sb, x_sl, x_sh}, dtype, g, cs, ddA_next, raw, d,
                           as_stream(stream));
}

int ema_chunk_scan_bwd_dc(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, int dtype,
                          const float* prev, const float* cs, float* ddA_prev, int64_t batch,
                          int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk,
                          void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  if (!cs || !ddA_prev) return EMA_ERR_NULL;
  EMA_TRY(check_f32(prev));
  return launch_row_dot<1>(dy, SeqStrides{dy_sb, dy_sl, dy_sh}, dtype, prev, cs, ddA_prev, 0, d,
                           as_stream(stream));
}

size_t ema_chunk_scan_bwd_ddAcs_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen,
                                                int64_t dim, int64_t chunk, int dtype) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, chunk, true, &d) != EMA_OK) return 0;
  if (check_dtype(dtype) != EMA_OK) return 0;
  return carve_da(nullptr, d, dtype).bytes;
}

int ema_chunk_scan_bwd_ddAcs(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                             const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, int dtype,
                             const float* cs, float* ddA_intra, void* workspace,
                             size_t workspace_bytes, int64_t batch, int64_t nheads, int64_t seqlen,
                             int64_t dim, int64_t chunk, void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  if (!cs || !ddA_intra) return EMA_ERR_NULL;
  EMA_TRY(check_f32(workspace));
  const DaWs w = carve_da(workspace, d, dtype);
  if (workspace_bytes < w.bytes) return EMA_ERR_SHAPE;
  return launch_da(x, SeqStrides{x_sb, x_sl, x_sh}, dy, SeqStrides{dy_sb, dy_sl, dy_sh}, dtype, cs,
                   ddA_intra, w, d, as_stream(stream));
}

// Workspace of ema_bwd: the chained part first, then the dA partials and what the recomputation
// of the chunk-entry states needs.
struct BwdWs {
  void* chain;
  float *cs, *states, *prev, *part;
  size_t bytes;
};
static BwdWs carve_bwd(void* base, const Dims& di) {
  BwdWs w;
  size_t off = chain_ws_bytes(di);
  char* p = static_cast<char*>(base);
  w.chain = base;
  auto take = [&](size_t floats) {
    float* r = reinterpret_cast<float*>(p + off);
    off += align_up(floats * sizeof(float), 256);
    return r;
  };
  const size_t ncq = (size_t)(di.N * di.C * di.Q), nct = (size_t)(di.N * di.C * di.T);
  w.cs = take(ncq);
  w.states = take(nct);
  w.prev = take(nct);
  const int parts_bf16 = tile_parts_per_dim<TileBf16>(di.T), parts_f32 = tile_parts_per_dim<TileF32>(di.T);
  w.part = take(ncq * (size_t)(parts_bf16 > parts_f32 ? parts_bf16 : parts_f32));
  w.bytes = off;
  return w;
}

size_t ema_bwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                               int64_t chunk) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, chunk, true, &d) != EMA_OK) return 0;
  return carve_bwd(nullptr, internal_dims(d)).bytes;
}

int ema_bwd(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, const void* x,
            int64_t x_sb, int64_t x_sl, int64_t x_sh, const float* A, int64_t a_sb, int64_t a_sl,
            int64_t a_sh, const float* prev128, int dtype, void* dx, int64_t dx_sb, int64_t dx_sl,
            int64_t dx_sh, float* ddA, void* y, int64_t y_sb, int64_t y_sl, int64_t y_sh,
            void* workspace, size_t workspace_bytes, int workspace_ready, int64_t batch, int64_t nheads,
            int64_t seqlen, int64_t dim, int64_t chunk, void* stream, void* ev_start, void* ev_stop) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, chunk, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(dx, dx_sb, dx_sl, dx_sh, dtype, dim));
  if (y) EMA_TRY(check_seq(y, y_sb, y_sl, y_sh, dtype, dim));
  if (!A || !ddA) return EMA_ERR_NULL;
  EMA_TRY(check_f32(workspace));
  if (workspace_bytes < ema_bwd_workspace_bytes(batch, nheads, seqlen, dim, chunk))
    return EMA_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  // The gradients do not depend on how the sequence is chunked, so the backward always
  // works on 128-row chunks (one tile of the kernel); `chunk` only fixes the (N, C, Q)
  // layout in which ddA is returned.
  const Dims di = internal_dims(d);
  const BwdWs w = carve_bwd(workspace, di);
  const SeqStrides sx{x_sb, x_sl, x_sh}, sd{dy_sb, dy_sl, dy_sh}, sdx{dx_sb, dx_sl, dx_sh};
  const SeqStrides sy{y_sb, y_sl, y_sh};

  const SeqStrides sa{a_sb, a_sl, a_sh};
  if (!prev128) {
    // states entering each chunk, recomputed: chunk states, then the inter-chunk recurrence
    // (its final state is not needed and lands in `part`, which is free until the main kernel)
    EMA_TRY(launch_cumsum(A, sa, w.cs, di, st));
    EMA_TRY(launch_chunk_reduce<0>(x, sx, dtype, w.cs, w.states, di, st));
    EMA_TRY(launch_state_passing_fwd(w.states, w.cs + (di.Q - 1), di.C * di.Q, di.Q, w.prev,
                                     w.part, di.N, di.C, di.T, st));
    prev128 = w.prev;
  }
  // dx, the recomputed y and the per-column-tile partials of dA in one pass over x and dy;
  // the reverse inter-chunk state is handed over inside the kernel
  int parts = dtype == EMA_BF16 ? tile_parts_per_dim<TileBf16>(di.T) : tile_parts_per_dim<TileF32>(di.T);
  if (dtype == EMA_BF16) {
    EMA_TRY((launch_bwd_tile_t<bf16_t, TileBf16, false>(x, sx, dy, sd, A, sa, prev128, dx, sdx, y, sy, w.part,
                                                        nullptr, nullptr, w.chain, workspace_ready != 0, di,
                                                        st, ev_start, ev_stop)));
  } else
    EMA_TRY((launch_bwd_tile_t<float, TileF32, false>(x, sx, dy, sd, A, sa, prev128, dx, sdx, y, sy, w.part,
                                                      nullptr, nullptr, w.chain, workspace_ready != 0, di, st,
                                                      ev_start, ev_stop)));
  const int64_t total = d.N * d.C * d.Q;
  hipLaunchKernelGGL(dA_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w.part,
                     ddA, (int)d.L, (int)d.Q, (int)d.C, (int)di.C, parts, total);
  return launched();
}

size_t ema_bwd_dx_dA_fused_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen,
                                           int64_t dim) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d) != EMA_OK) return 0;
  return align_up((size_t)(d.N * d.C * d.Q) * bwd_col_tiles(d, EMA_F32) * sizeof(float), 256);
}

int ema_bwd_dx_dA_fused(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, const void* dy,
                        int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, int dtype, const float* cs,
                        const float* prev, const float* g, void* dx, int64_t dx_sb, int64_t dx_sl,
                        int64_t dx_sh, float* ddA, void* y, int64_t y_sb, int64_t y_sl, int64_t y_sh,
                        void* workspace, size_t workspace_bytes, int64_t batch, int64_t nheads,
                        int64_t seqlen, int64_t dim, void* stream) {
  Dims d;
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  EMA_TRY(check_seq(dx, dx_sb, dx_sl, dx_sh, dtype, dim));
  if (y) EMA_TRY(check_seq(y, y_sb, y_sl, y_sh, dtype, dim));
  if (!cs || !ddA) return EMA_ERR_NULL;
  EMA_TRY(check_f32(prev));
  EMA_TRY(check_f32(g));
  EMA_TRY(check_f32(workspace));
  if (workspace_bytes < ema_bwd_dx_dA_fused_workspace_bytes(batch, nheads, seqlen, dim))
    return EMA_ERR_SHAPE;
  return run_bwd_fused(x, SeqStrides{x_sb, x_sl, x_sh}, dy, SeqStrides{dy_sb, dy_sl, dy_sh}, dtype, cs,
                       prev, g, dx, SeqStrides{dx_sb, dx_sl, dx_sh}, y, SeqStrides{y_sb, y_sl, y_sh},
                       ddA, static_cast<float*>(workspace), d, d, as_stream(stream));
}

// ---- sequence-level entry points: either form of the recurrence, optional boundary states

static int check_form(int form) {
  return (form == EMA_FORM_LOG_DECAY || form == EMA_FORM_PROBABILITY) ? EMA_OK : EMA_ERR_UNSUPPORTED;
}

size_t ema_seq_fwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d) != EMA_OK) return 0;
  return carve_seq(nullptr, d, false).bytes;
}

static int seq_fwd_impl(int form, const float* coef, int64_t c_sb, int64_t c_sl, int64_t c_sh, const void* x,
                        int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y, int64_t y_sb,
                        int64_t y_sl, int64_t y_sh, const float* init, float* final_state, float* prev128,
                        void* workspace, size_t workspace_bytes, int workspace_ready, int64_t batch,
                        int64_t nheads, int64_t seqlen, int64_t dim, void* stream, void* ev_start,
                        void* ev_stop) {
  Dims d;
  EMA_TRY(check_form(form));
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(y, y_sb, y_sl, y_sh, dtype, dim));
  if (!coef || !prev128) return EMA_ERR_NULL;
  EMA_TRY(check_f32(workspace));
  if (workspace_bytes < ema_seq_fwd_workspace_bytes(batch, nheads, seqlen, dim)) return EMA_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  const SeqWs w = carve_seq(workspace, d, false);
  const SeqStrides sx{x_sb, x_sl, x_sh}, sy{y_sb, y_sl, y_sh}, sc{c_sb, c_sl, c_sh};
  const bool xp = form == EMA_FORM_PROBABILITY, ready = workspace_ready != 0;
  if (dtype == EMA_BF16) {
    if (xp)
      return launch_fwd_tile_t<bf16_t, TileBf16, true>(x, sx, coef, sc, y, sy, prev128, nullptr, 1, final_state,
                                                       init, w.chain, ready, d, st, ev_start, ev_stop);
    return launch_fwd_tile_t<bf16_t, TileBf16, false>(x, sx, coef, sc, y, sy, prev128, nullptr, 1, final_state,
                                                      init, w.chain, ready, d, st, ev_start, ev_stop);
  }
  if (xp)
    return launch_fwd_tile_t<float, TileF32, true>(x, sx, coef, sc, y, sy, prev128, nullptr, 1, final_state, init,
                                                   w.chain, ready, d, st, ev_start, ev_stop);
  return launch_fwd_tile_t<float, TileF32, false>(x, sx, coef, sc, y, sy, prev128, nullptr, 1, final_state, init,
                                                  w.chain, ready, d, st, ev_start, ev_stop);
}

int ema_seq_fwd(int form, const float* coef, int64_t c_sb, int64_t c_sl, int64_t c_sh, const void* x,
                int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y, int64_t y_sb,
                int64_t y_sl, int64_t y_sh, const float* init, float* final_state, float* prev128,
                void* workspace, size_t workspace_bytes, int workspace_ready, int64_t batch, int64_t nheads,
                int64_t seqlen, int64_t dim, void* stream, void* ev_start, void* ev_stop) {
  return seq_fwd_impl(form, coef, c_sb, c_sl, c_sh, x, x_sb, x_sl, x_sh, dtype, y, y_sb, y_sl, y_sh, init,
                      final_state, prev128, workspace, workspace_bytes, workspace_ready, batch, nheads, seqlen,
                      dim, stream, ev_start, ev_stop);
}

// ---- the entry point that allocates nothing: ema_seq_fwd with its workspace in a file-scope array

size_t ema_seq_fwd_static_max_workspace_bytes(void) { return kScratchBytes; }

int ema_seq_fwd_static(int form, const float* coef, int64_t c_sb, int64_t c_sl, int64_t c_sh, const void* x,
                       int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y, int64_t y_sb,
                       int64_t y_sl, int64_t y_sh, const float* init, float* final_state, float* prev128,
                       int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, void* stream) {
  const size_t need = ema_seq_fwd_workspace_bytes(batch, nheads, seqlen, dim);
  if (need == 0) return EMA_ERR_SHAPE;
  if (need > kScratchBytes) return EMA_ERR_TOO_LARGE;
  void* ws = nullptr;
  EMA_TRY(scratch_address(&ws));
  // the array starts out zero-filled and is only ever written by this entry point's kernels,
  // which leave it ready for the next call: nothing has to be cleared
  return seq_fwd_impl(form, coef, c_sb, c_sl, c_sh, x, x_sb, x_sl, x_sh, dtype, y, y_sb, y_sl, y_sh, init,
                      final_state, prev128, ws, kScratchBytes, 1, batch, nheads, seqlen, dim, stream, nullptr,
                      nullptr);
}

int ema_seq_fwd_static_init(void) {
  void* ws = nullptr;
  return scratch_address(&ws);
}

int ema_seq_fwd_static_error(int* error, void* stream) {
  if (!error) return EMA_ERR_NULL;
  void* ws = nullptr;
  EMA_TRY(scratch_address(&ws));
  hipStream_t st = as_stream(stream);
  unsigned word = 0;
  const unsigned* src = &static_cast<const ChainHeader*>(ws)->error;
  if (hipMemcpyAsync(&word, src, sizeof(word), hipMemcpyDeviceToHost, st) != hipSuccess ||
      hipStreamSynchronize(st) != hipSuccess)
    return EMA_ERR_LAUNCH;
  *error = (int)word;
  return EMA_OK;
}

int ema_seq_fwd_static_reset(void* stream) {
  void* ws = nullptr;
  EMA_TRY(scratch_address(&ws));
  return launch_clear(ws, kScratchBytes, as_stream(stream));
}

size_t ema_seq_bwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim) {
  Dims d;
  if (check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d) != EMA_OK) return 0;
  return carve_seq(nullptr, d, true).bytes;
}

int ema_seq_bwd(int form, const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, const void* x,
                int64_t x_sb, int64_t x_sl, int64_t x_sh, const float* coef, int64_t c_sb, int64_t c_sl,
                int64_t c_sh, const float* prev128, const float* dfinal, int dtype, void* dx,
                int64_t dx_sb, int64_t dx_sl, int64_t dx_sh, float* dcoef, int64_t dc_sb, int64_t dc_sl,
                int64_t dc_sh, float* dinit, void* workspace, size_t workspace_bytes, int workspace_ready,
                int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, void* stream, void* ev_start,
                void* ev_stop) {
  Dims d;
  EMA_TRY(check_form(form));
  EMA_TRY(check_dims(batch, nheads, seqlen, dim, kTileRows, true, &d));
  EMA_TRY(check_dtype(dtype));
  EMA_TRY(check_seq(dy, dy_sb, dy_sl, dy_sh, dtype, dim));
  EMA_TRY(check_seq(x, x_sb, x_sl, x_sh, dtype, dim));
  EMA_TRY(check_seq(dx, dx_sb, dx_sl, dx_sh, dtype, dim));
  if (!coef || !prev128 || !dcoef) return EMA_ERR_NULL;
  EMA_TRY(check_f32(workspace));
  if (workspace_bytes < ema_seq_bwd_workspace_bytes(batch, nheads, seqlen, dim)) return EMA_ERR_SHAPE;
  const bool ready = workspace_ready != 0;
  hipStream_t st = as_stream(stream);
  const SeqWs w = carve_seq(workspace, d, true);
  const SeqStrides sx{x_sb, x_sl, x_sh}, sd{dy_sb, dy_sl, dy_sh}, sdx{dx_sb, dx_sl, dx_sh};
  const SeqStrides sc{c_sb, c_sl, c_sh}, none{0, 0, 0};
  const bool xp = form == EMA_FORM_PROBABILITY;
  int parts;
  if (dtype == EMA_BF16) {
    parts = tile_parts_per_dim<TileBf16>(d.T);
    if (xp)
      EMA_TRY((launch_bwd_tile_t<bf16_t, TileBf16, true>(x, sx, dy, sd, coef, sc, prev128, dx, sdx, nullptr, none,
                                                         w.part, dfinal, dinit, w.chain, ready, d, st, ev_start,
                                                         ev_stop)));
    else
      EMA_TRY((launch_bwd_tile_t<bf16_t, TileBf16, false>(x, sx, dy, sd, coef, sc, prev128, dx, sdx, nullptr, none,
                                                          w.part, dfinal, dinit, w.chain, ready, d, st, ev_start,
                                                          ev_stop)));
  } else {
    parts = tile_parts_per_dim<TileF32>(d.T);
    if (xp)
      EMA_TRY((launch_bwd_tile_t<float, TileF32, true>(x, sx, dy, sd, coef, sc, prev128, dx, sdx, nullptr, none,
                                                       w.part, dfinal, dinit, w.chain, ready, d, st, ev_start,
                                                       ev_stop)));
    else
      EMA_TRY((launch_bwd_tile_t<float, TileF32, false>(x, sx, dy, sd, coef, sc, prev128, dx, sdx, nullptr, none,
                                                        w.part, dfinal, dinit, w.chain, ready, d, st, ev_start,
                                                        ev_stop)));
  }
  const int64_t total = d.N * d.L;
  hipLaunchKernelGGL(dcoef_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w.part,
                     dcoef, SeqStrides{dc_sb, dc_sl, dc_sh}, (int)d.nh, (int)d.L, (int)d.C, parts, total);
  return launched();
}

#ifdef EMA_TIMING
// Development aid, only in builds with -DEMA_TIMING: installs the per-tile timestamp buffer.
int ema_debug_set_timing(void* buf) {
  return hipMemcpyToSymbol(HIP_SYMBOL(ema::g_ema_timing), &buf, sizeof(buf)) == hipSuccess ? 0 : -6;
}
#endif

}  // extern "C"
