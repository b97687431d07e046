// C ABI of the SSD forward stages: argument validation and kernel launches.  Declarations and
// the reference launcher each entry point replaces are in include/ssd_hip.h.
#include "../../include/ssd_hip.h"

#include <hip/hip_runtime.h>

#include <type_traits>

#include "ema_gemm_kernels.h"
#include "ssd_kernels.h"

using namespace ssd;

namespace {

#define SSD_TRY(expr)            \
  do {                           \
    int _s = (expr);             \
    if (_s != SSD_OK) return _s; \
  } while (0)

inline int launched() { return hipGetLastError() == hipSuccess ? SSD_OK : SSD_ERR_LAUNCH; }
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline int esize(int dtype) { return dtype == SSD_BF16 ? 2 : 4; }
inline int check_dtype(int dtype) { return (dtype == SSD_F32 || dtype == SSD_BF16) ? SSD_OK : SSD_ERR_DTYPE; }

// A tensor read or written in 16-byte pieces along its dense last axis of `inner` elements.
int check_vec(const void* p, int64_t sb, int64_t sl, int64_t sh, int dtype, int64_t inner) {
  if (!p) return SSD_ERR_NULL;
  const int epl = 16 / esize(dtype);
  if (inner % epl || sb % epl || sl % epl || sh % epl) return SSD_ERR_ALIGN;
  if (reinterpret_cast<uintptr_t>(p) % 16) return SSD_ERR_ALIGN;
  return SSD_OK;
}
int check_f32(const void* p) {
  if (!p) return SSD_ERR_NULL;
  return reinterpret_cast<uintptr_t>(p) % 16 ? SSD_ERR_ALIGN : SSD_OK;
}

// The kernels that copy their operands straight into LDS form 32-bit unsigned byte offsets from
// the strides: tensors addressed with a negative stride go to the register-staged kernels.
inline bool forward_strides(const Strides3& s) { return s.sb >= 0 && s.sl >= 0 && s.sh >= 0; }

// A carried-state tensor is float32 or of the inputs' type (16-byte aligned either way).
int check_state(const void* p, int state_dtype, int dtype) {
  if (state_dtype != SSD_F32 && state_dtype != dtype) return SSD_ERR_DTYPE;
  return check_f32(p);
}

struct Dims {
  int64_t batch, L, nh, g, P, N, Q, C;
};
int check_dims(int64_t batch, int64_t L, int64_t nh, int64_t g, int64_t P, int64_t N, int64_t Q, Dims* d) {
  if (batch <= 0 || L <= 0 || nh <= 0 || g <= 0 || Q <= 0) return SSD_ERR_SHAPE;
  if (nh % g) return SSD_ERR_SHAPE;
  if (Q > 1024 || Q % 4) return SSD_ERR_UNSUPPORTED;
  if (batch > (1 << 20) || nh > (1 << 16) || L > ((int64_t)1 << 30)) return SSD_ERR_SHAPE;
  *d = Dims{batch, L, nh, g, P, N, Q, (L + Q - 1) / Q};
  if (batch * nh * d->C > ((int64_t)1 << 28)) return SSD_ERR_SHAPE;
  return SSD_OK;
}
inline bool dim_ok(int64_t v) { return v == 64 || v == 128; }
// The state-passing entries take the chunking only to locate the last position of each chunk of
// a packed batch; without seq_idx both numbers are ignored.
inline int check_seq_chunks(const int32_t* seq_idx, int64_t seqlen, int64_t chunk, int64_t nchunks) {
  if (!seq_idx) return SSD_OK;
  if (seqlen <= 0 || chunk <= 0 || seqlen > ((int64_t)1 << 30)) return SSD_ERR_SHAPE;
  return (seqlen + chunk - 1) / chunk == nchunks ? SSD_OK : SSD_ERR_SHAPE;
}
inline SeqIdx as_seq(const int32_t* p, int64_t sb, int64_t sl) { return SeqIdx{p, sb, sl}; }
constexpr int kLdsBytes = 160 * 1024;  // LDS of one CU

template <typename K>
int allow_smem(K kernel, int bytes) {
  if (bytes <= 64 * 1024) return SSD_OK;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             bytes) == hipSuccess
             ? SSD_OK
             : SSD_ERR_LAUNCH;
}

// Calls f.template run<T, P, N>() for the runtime (dtype, hdim, dstate).
template <typename F>
int dispatch_tpn(int dtype, int64_t P, int64_t N, F f) {
  if (dtype == SSD_BF16) {
    if (P == 64 && N == 64) return f.template run<bf16_t, 64, 64>();
    if (P == 64 && N == 128) return f.template run<bf16_t, 64, 128>();
    if (P == 128 && N == 64) return f.template run<bf16_t, 128, 64>();
    return f.template run<bf16_t, 128, 128>();
  }
  if (P == 64 && N == 64) return f.template run<float, 64, 64>();
  if (P == 64 && N == 128) return f.template run<float, 64, 128>();
  if (P == 128 && N == 64) return f.template run<float, 128, 64>();
  return f.template run<float, 128, 128>();
}

template <int MODE>
struct StateLaunch {
  const void *x, *B;
  Strides3 sx, sB;
  const float *dt, *dA;
  void* states;
  int states_dtype;
  Dims d;
  SeqIdx seq;
  hipStream_t st;
  template <typename T, int P, int N>
  int run() const {
    if constexpr (!std::is_same<T, float>::value)
      if (states_dtype != SSD_F32) return run_as<T, P, N, T>();
    return run_as<T, P, N, float>();
  }
  template <typename T, int P, int N, typename TO>
  int run_as() const {
    auto kernel = ssd_chunk_state_kernel<T, P, N, MODE, TO>;
    constexpr int smem = StateSmem<T, P, N>::kBytes;
    SSD_TRY(allow_smem(kernel, smem));
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.nh)), dim3(256), smem, st, (const T*)x, sx,
                       (const T*)B, sB, dt, dA, (TO*)states, (int)d.nh, (int)(d.nh / d.g), (int)d.L, (int)d.Q,
                       (int)d.C, seq);
    return launched();
  }
};

struct WalkLaunch {
  const void *x, *B;
  Strides3 sx, sB;
  const float *dt, *dA, *initial;
  void* out;
  int out_dtype;
  float* final_states;
  Dims d;
  hipStream_t st;
  template <typename T, int P, int N>
  int run() const {
    if (out_dtype == SSD_BF16) return run_as<T, P, N, bf16_t>();
    return run_as<T, P, N, float>();
  }
  template <typename T, int P, int N, typename TO>
  int run_as() const {
#ifndef SSD_WALK_DMA  // 0: development builds without the kernel that copies its rows straight into LDS
#define SSD_WALK_DMA 1
#endif
    // (the kernel keeps the byte offset of a row inside a stage in 32 bits)
    if constexpr (SSD_WALK_DMA && std::is_same<T, bf16_t>::value && P == 64 && N == 128) {
      if (forward_strides(sx) && forward_strides(sB) && sx.sl < (int64_t(1) << 24) && sB.sl < (int64_t(1) << 24)) {
        auto kernel = ssd_state_walk_dma_kernel<TO>;
        constexpr int smem = WalkDmaSmem::kBytes;
        SSD_TRY(allow_smem(kernel, smem));
        hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.nh)), dim3(512), smem, st, (const bf16_t*)x, sx,
                           (const bf16_t*)B, sB, dt, dA, initial, (TO*)out, final_states, (int)d.nh, (int)(d.nh / d.g),
                           (int)d.L, (int)d.Q, (int)d.C);
        return launched();
      }
    }
#ifndef SSD_WALK_NSPLIT  // 2: two workgroups per (b, h), half the state columns each (measured no faster: x crosses the L2 twice)
#define SSD_WALK_NSPLIT 1
#endif
    constexpr int NSPLIT = (SSD_WALK_NSPLIT == 2 && ((P / 32) * (N / 64)) % 4 == 0 && P * N <= 64 * 128) ? 2 : 1;
    auto kernel = ssd_state_walk_kernel<T, P, N, TO, NSPLIT>;
    constexpr int smem = WalkSmem<T, P, N / NSPLIT>::kBytes;
    SSD_TRY(allow_smem(kernel, smem));
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.nh * NSPLIT)), dim3(256), smem, st, (const T*)x, sx,
                       (const T*)B, sB, dt, dA, initial, (TO*)out, final_states, (int)d.nh, (int)(d.nh / d.g),
                       (int)d.L, (int)d.Q, (int)d.C);
    return launched();
  }
};

struct ScanLaunch {
  const float* cb;
  const void *x, *z, *C;
  Strides3 sx, sz, sC, so;
  const float *dt, *dA;
  const void* prev;
  int prev_dtype;
  const float* D;
  int d_has_hdim;
  void *out, *out_x;
  Dims d;
  SeqIdx seq;
  hipStream_t st;
  template <typename T, int P, int N>
  int run() const {
    if constexpr (!std::is_same<T, float>::value)
      if (prev_dtype != SSD_F32) return run_as<T, P, N, T>();
    return run_as<T, P, N, float>();
  }
  template <typename T, int P, int N, typename TS, int HP>
  int launch_wide() const {
    auto kernel = ssd_chunk_scan_wide_kernel<T, P, N, TS, HP>;
    constexpr int smem = WideSmem<T, P * HP, N>::bytes_for(HP);
    SSD_TRY(allow_smem(kernel, smem));
    const int stiles = (int)(d.Q / 256);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * (d.nh / HP) * stiles)), dim3(256), smem, st, cb,
                       (const T*)x, sx, (const T*)z, sz, dt, dA, (const T*)C, sC, (const TS*)prev, D, d_has_hdim,
                       (T*)out, so, (T*)out_x, (int)d.nh, (int)(d.nh / d.g), (int)d.g, (int)d.L, (int)d.Q, (int)d.C,
                       stiles, seq);
    return launched();
  }
  template <typename T, int P, int N, typename TS>
  int run_as() const {
    constexpr int wide_smem = WideSmem<T, P, N>::kBytes;
    if (d.Q % 256 == 0 && wide_smem <= kLdsBytes) {  // 256-row super-tiles, no barrier inside the k loop
      // Two adjacent heads of a group per workgroup where they are adjacent in memory too (dense
      // heads of 64 features): they share the fragments of cb and the rows of C.
      if constexpr (P == 64 && WideSmem<T, 128, N>::bytes_for(2) <= kLdsBytes / 2) {
        const bool dense = sx.sh == P && so.sh == P && (!z || sz.sh == P);
        if (dense && (d.nh / d.g) % 2 == 0) return launch_wide<T, P, N, TS, 2>();
      }
      return launch_wide<T, P, N, TS, 1>();
    }
    auto kernel = ssd_chunk_scan_kernel<T, P, N, TS>;
    constexpr int smem = ScanSmem<T, P, N>::kBytes;
    SSD_TRY(allow_smem(kernel, smem));
    const int mtiles = (int)((d.Q + 63) / 64);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.nh * mtiles)), dim3(256), smem, st, cb,
                       (const T*)x, sx, (const T*)z, sz, dt, dA, (const T*)C, sC, (const TS*)prev, D, d_has_hdim,
                       (T*)out, so, (T*)out_x, (int)d.nh, (int)(d.nh / d.g), (int)d.g, (int)d.L, (int)d.Q, (int)d.C, mtiles,
                       seq);
    return launched();
  }
};

struct DxLaunch {
  const float* cb;
  const void *x, *dout, *B;
  Strides3 sx, sd, sB, sdx;
  const float *dt, *dA;
  const void* dstates;
  int states_dtype;
  const float* D;
  int d_has_hdim;
  void* dx;
  float* ddt;
  Dims d;
  SeqIdx seq;
  float* dD_part;
  hipStream_t st;
  // whether the 256-row kernel runs this shape (it must also fit the LDS of a CU)
  template <typename T, int P, int N>
  static bool wide(int64_t Q) {
    return Q % 256 == 0 && WideSmem<T, P, N>::kBytes <= kLdsBytes;
  }
  template <typename T, int P, int N>
  int run() const {
    if constexpr (!std::is_same<T, float>::value)
      if (states_dtype != SSD_F32) return run_as<T, P, N, T>();
    return run_as<T, P, N, float>();
  }
  template <typename T, int P, int N, typename TS>
  int run_as() const {
    constexpr int wide_smem = WideSmem<T, P, N>::kBytes;
    if (wide<T, P, N>(d.Q)) {
      auto kernel = ssd_chunk_scan_bwd_dx_wide_kernel<T, P, N, TS>;
      SSD_TRY(allow_smem(kernel, wide_smem));
      const int stiles = (int)(d.Q / 256);
      hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.nh * stiles)), dim3(256), wide_smem, st, cb,
                         (const T*)x, sx, (const T*)dout, sd, dt, dA, (const T*)B, sB, (const TS*)dstates, D,
                         d_has_hdim, (T*)dx, sdx, ddt, (int)d.nh, (int)(d.nh / d.g), (int)d.g, (int)d.L, (int)d.Q,
                         (int)d.C, stiles, seq, dD_part);
      return launched();
    }
    auto kernel = ssd_chunk_scan_bwd_dx_kernel<T, P, N, TS>;
    constexpr int smem = ScanSmem<T, P, N>::kBytes;
    SSD_TRY(allow_smem(kernel, smem));
    const int mtiles = (int)((d.Q + 63) / 64);
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.nh * mtiles)), dim3(256), smem, st, cb,
                       (const T*)x, sx, (const T*)dout, sd, dt, dA, (const T*)B, sB, (const TS*)dstates, D, d_has_hdim,
                       (T*)dx, sdx, ddt, (int)d.nh, (int)(d.nh / d.g), (int)d.g, (int)d.L, (int)d.Q, (int)d.C, mtiles,
                       seq, dD_part);
    return launched();
  }
};

// Number of per-wave slots the dx kernel of a shape writes per (batch, chunk, head).
struct DxSlots {
  int64_t Q;
  template <typename T, int P, int N>
  int run() const {
    return DxLaunch::wide<T, P, N>(Q) ? (int)(4 * (Q / 256)) : (int)(4 * ((Q + 63) / 64));
  }
};

template <int MODE>
struct GroupLaunch {
  const void* a;
  Strides3 sa;
  const void* s;
  int s_dtype;
  const float *dt, *dA;
  const void* bc;
  Strides3 sbc;
  float *out, *ddA;
  Dims d;
  SeqIdx seq;
  hipStream_t st;
  template <typename T, int P, int N>
  int run() const {
    if constexpr (!std::is_same<T, float>::value)
      if (s_dtype != SSD_F32) return run_as<T, P, N, T>();
    return run_as<T, P, N, float>();
  }
  template <typename T, int P, int N, typename TS>
  int run_as() const {
#ifndef SSD_GROUP_DMA  // 0: development builds without the kernel that copies its operands straight into LDS
#define SSD_GROUP_DMA 1
#endif
    if constexpr (SSD_GROUP_DMA && std::is_same<T, bf16_t>::value && std::is_same<TS, bf16_t>::value && P == 64 && N == 128) {
      // (the kernel keeps the byte offset of a row inside a chunk in 32 bits)
      if (d.Q % 64 == 0 && !seq.p && forward_strides(sa) && forward_strides(sbc) && d.Q * sa.sl < (int64_t(1) << 30)) {
        auto kernel = ssd_group_grad_dma_kernel<MODE>;
        constexpr int smem = GroupDmaSmem::kBytes;
        SSD_TRY(allow_smem(kernel, smem));
        const int mtiles = (int)(d.Q / 64);
        if (d.batch * d.C * d.g * mtiles > 0x7fffffff) return SSD_ERR_SHAPE;
        hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.g * mtiles)), dim3(256), smem, st, (const bf16_t*)a,
                           sa, (const bf16_t*)s, dt, dA, (const bf16_t*)bc, sbc, out, ddA, (int)d.nh, (int)(d.nh / d.g),
                           (int)d.g, (int)d.L, (int)d.Q, (int)d.C, mtiles);
        return launched();
      }
    }
    auto kernel = ssd_group_grad_kernel<T, P, N, MODE, TS>;
    constexpr int smem = GroupSmem<T, P, N>::kBytes;
    SSD_TRY(allow_smem(kernel, smem));
    const int mtiles = (int)((d.Q + 63) / 64);
    if (d.batch * d.C * d.g * mtiles > 0x7fffffff) return SSD_ERR_SHAPE;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(d.batch * d.C * d.g * mtiles)), dim3(256), smem, st, (const T*)a, sa,
                       (const TS*)s, dt, dA, (const T*)bc, sbc, out, ddA, (int)d.nh, (int)(d.nh / d.g), (int)d.g, (int)d.L,
                       (int)d.Q, (int)d.C, mtiles, seq);
    return launched();
  }
};

int launch_row_cumsum(float* v, int64_t Q, int64_t rows, hipStream_t st) {
  hipLaunchKernelGGL(ssd_row_cumsum_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, v, (int)Q, rows);
  return launched();
}

template <typename T, typename TO, int K>
int launch_bmm(const void* a, Strides3 sa, const void* bm, Strides3 sb, void* out, const Dims& d, SeqIdx seq,
               hipStream_t st) {
  auto kernel = ssd_bmm_kernel<T, TO, K>;
  constexpr int smem = bmm_smem_bytes<T, K>();
  SSD_TRY(allow_smem(kernel, smem));
  const int tiles = (int)((d.Q + 63) / 64);
  const int64_t grid = d.batch * d.C * d.g * tiles * tiles;
  if (grid > 0x7fffffff) return SSD_ERR_SHAPE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), smem, st, (const T*)a, sa, (const T*)bm, sb, (TO*)out,
                     (int)d.g, (int)d.L, (int)d.Q, (int)d.C, tiles, seq);
  return launched();
}

}  // namespace

extern "C" {

int ssd_chunk_cumsum_fwd(const void* dt, int dt_dtype, int64_t dt_sb, int64_t dt_sl, int64_t dt_sh,
                         const float* A, const float* dt_bias, float* dA_cumsum, float* dt_out,
                         int64_t batch, int64_t seqlen, int64_t nheads, int64_t chunk, int dt_softplus,
                         float dt_min, float dt_max, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, 1, 0, 0, chunk, &d));
  SSD_TRY(check_dtype(dt_dtype));
  if (!dt || !A || !dA_cumsum || !dt_out) return SSD_ERR_NULL;
  const Strides3 sd{dt_sb, dt_sl, dt_sh};
  // heads per workgroup: a power of two up to 8 (32-byte pieces of dt rows; more heads per workgroup
  // leave too few workgroups to hide their latency) whose Q x HT tile stays within 64 KB of LDS
  int HT = 8;
  while (HT > 1 && (HT / 2 >= nheads || (int64_t)HT * (chunk + 1) * 4 > 64 * 1024)) HT /= 2;
  const int hgroups = (int)((nheads + HT - 1) / HT);
  const int64_t blocks = batch * d.C * hgroups;
  if (blocks > 0x7fffffff) return SSD_ERR_SHAPE;
  const unsigned grid = (unsigned)blocks;
  const int smem = HT * (int)(chunk + 1) * 4;
  if (dt_dtype == SSD_BF16)
    hipLaunchKernelGGL(ssd_cumsum_kernel<bf16_t>, dim3(grid), dim3(256), smem, as_stream(stream), (const bf16_t*)dt,
                       sd, A, dt_bias, dA_cumsum, dt_out, (int)nheads, (int)seqlen, (int)chunk, (int)d.C, dt_softplus,
                       dt_min, dt_max, HT, hgroups);
  else
    hipLaunchKernelGGL(ssd_cumsum_kernel<float>, dim3(grid), dim3(256), smem, as_stream(stream), (const float*)dt, sd,
                       A, dt_bias, dA_cumsum, dt_out, (int)nheads, (int)seqlen, (int)chunk, (int)d.C, dt_softplus,
                       dt_min, dt_max, HT, hgroups);
  return launched();
}

int ssd_chunk_state_fwd(const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, const void* x,
                        int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, const float* dt,
                        const float* dA_cumsum, float* states, int64_t batch, int64_t seqlen,
                        int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                        const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  SSD_TRY(check_vec(B, b_sb, b_sl, b_sg, dtype, dstate));
  if (!dt || !dA_cumsum) return SSD_ERR_NULL;
  SSD_TRY(check_f32(states));
  return dispatch_tpn(dtype, hdim, dstate,
                      StateLaunch<0>{x, B, Strides3{x_sb, x_sl, x_sh}, Strides3{b_sb, b_sl, b_sg}, dt, dA_cumsum,
                                     states, SSD_F32, d, as_seq(seq_idx, seq_sb, seq_sl), as_stream(stream)});
}

int ssd_chunk_state_passing_fwd(const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, const void* x,
                                int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, const float* dt,
                                const float* dA_cumsum, const float* initial, void* out, int out_dtype,
                                float* final_states, int64_t batch, int64_t seqlen, int64_t nheads,
                                int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  SSD_TRY(check_dtype(out_dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate) || chunk % 64) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  SSD_TRY(check_vec(B, b_sb, b_sl, b_sg, dtype, dstate));
  SSD_TRY(check_f32(dt));  // fetched in 16-byte pieces
  SSD_TRY(check_f32(dA_cumsum));
  SSD_TRY(check_f32(out));
  SSD_TRY(check_f32(final_states));
  if (initial) SSD_TRY(check_f32(initial));
  return dispatch_tpn(dtype, hdim, dstate,
                      WalkLaunch{x, B, Strides3{x_sb, x_sl, x_sh}, Strides3{b_sb, b_sl, b_sg}, dt, dA_cumsum, initial,
                                 out, out_dtype, final_states, d, as_stream(stream)});
}

int ssd_state_passing_fwd(const float* states, const float* dA_chunk, int64_t da_sb, int64_t da_sh,
                          int64_t da_sc, const float* initial, void* out, int out_dtype, float* final_states,
                          int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim, const int32_t* seq_idx,
                          int64_t seq_sb, int64_t seq_sl, int64_t seqlen, int64_t chunk, void* stream) {
  if (batch <= 0 || nchunks <= 0 || nheads <= 0 || dim <= 0) return SSD_ERR_SHAPE;
  if (dim % 4) return SSD_ERR_ALIGN;
  if (!dA_chunk) return SSD_ERR_NULL;
  SSD_TRY(check_dtype(out_dtype));
  SSD_TRY(check_seq_chunks(seq_idx, seqlen, chunk, nchunks));
  SSD_TRY(check_f32(states));
  SSD_TRY(check_f32(out));
  SSD_TRY(check_f32(final_states));
  if (initial) SSD_TRY(check_f32(initial));
  // four elements per thread: 16-byte loads of the float32 states, 8-byte stores of a bfloat16 out
  // (eight per thread, which makes those stores 16 bytes, measured 8 % slower here)
  const int tiles = (int)((dim + 1023) / 1024);
  const int64_t grid = batch * nheads * tiles;
  if (grid > 0x7fffffff || dim > (1 << 24)) return SSD_ERR_SHAPE;
#define SSD_SP_LAUNCH(TO)                                                                                          \
  hipLaunchKernelGGL((ssd_state_passing_kernel<TO, 4>), dim3((unsigned)grid), dim3(256), 0, as_stream(stream), states, \
                     dA_chunk, da_sb, da_sh, da_sc, initial, (TO*)out, final_states, (int)nheads, (int)nchunks,      \
                     (int)dim, tiles, as_seq(seq_idx, seq_sb, seq_sl), (int)seqlen, (int)chunk)
  if (out_dtype == SSD_BF16) SSD_SP_LAUNCH(bf16_t);
  else SSD_SP_LAUNCH(float);
#undef SSD_SP_LAUNCH
  return launched();
}

int ssd_bmm_chunk_fwd(const void* a, int64_t a_sb, int64_t a_sl, int64_t a_sg, const void* bm,
                      int64_t b_sb, int64_t b_sl, int64_t b_sg, int dtype, void* out, int out_dtype,
                      int64_t batch, int64_t seqlen, int64_t ngroups, int64_t k, int64_t chunk,
                      const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, ngroups, ngroups, 0, k, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  SSD_TRY(check_dtype(out_dtype));
  if (!dim_ok(k)) return SSD_ERR_UNSUPPORTED;
  if (out_dtype != SSD_F32 && out_dtype != dtype) return SSD_ERR_DTYPE;
  SSD_TRY(check_vec(a, a_sb, a_sl, a_sg, dtype, k));
  SSD_TRY(check_vec(bm, b_sb, b_sl, b_sg, dtype, k));
  if (!out) return SSD_ERR_NULL;
  const Strides3 sa{a_sb, a_sl, a_sg}, sb{b_sb, b_sl, b_sg};
  hipStream_t st = as_stream(stream);
  const SeqIdx seq = as_seq(seq_idx, seq_sb, seq_sl);
  if (dtype == SSD_BF16) {
    if (out_dtype == SSD_F32)
      return k == 64 ? launch_bmm<bf16_t, float, 64>(a, sa, bm, sb, out, d, seq, st)
                     : launch_bmm<bf16_t, float, 128>(a, sa, bm, sb, out, d, seq, st);
    return k == 64 ? launch_bmm<bf16_t, bf16_t, 64>(a, sa, bm, sb, out, d, seq, st)
                   : launch_bmm<bf16_t, bf16_t, 128>(a, sa, bm, sb, out, d, seq, st);
  }
  return k == 64 ? launch_bmm<float, float, 64>(a, sa, bm, sb, out, d, seq, st)
                 : launch_bmm<float, float, 128>(a, sa, bm, sb, out, d, seq, st);
}

int ssd_chunk_scan_fwd(const float* cb, const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                       const void* z, int64_t z_sb, int64_t z_sl, int64_t z_sh, int dtype,
                       const float* dt, const float* dA_cumsum, const void* C, int64_t c_sb, int64_t c_sl,
                       int64_t c_sg, const void* prev_states, int states_dtype, const float* D, int d_has_hdim,
                       void* out, int64_t o_sb, int64_t o_sl, int64_t o_sh, void* out_x, int64_t batch,
                       int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate,
                       int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  SSD_TRY(check_vec(out, o_sb, o_sl, o_sh, dtype, hdim));
  SSD_TRY(check_vec(C, c_sb, c_sl, c_sg, dtype, dstate));
  if (z) SSD_TRY(check_vec(z, z_sb, z_sl, z_sh, dtype, hdim));
  if (out_x && reinterpret_cast<uintptr_t>(out_x) % 16) return SSD_ERR_ALIGN;
  if (!dt || !dA_cumsum) return SSD_ERR_NULL;
  SSD_TRY(check_f32(cb));
  SSD_TRY(check_state(prev_states, states_dtype, dtype));
  if (batch * d.C * nheads * ((chunk + 63) / 64) > 0x7fffffff) return SSD_ERR_SHAPE;
  return dispatch_tpn(dtype, hdim, dstate,
                      ScanLaunch{cb, x, z, C, Strides3{x_sb, x_sl, x_sh}, Strides3{z_sb, z_sl, z_sh},
                                 Strides3{c_sb, c_sl, c_sg}, Strides3{o_sb, o_sl, o_sh}, dt, dA_cumsum,
                                 prev_states, states_dtype, D, d_has_hdim, out, out_x, d,
                                 as_seq(seq_idx, seq_sb, seq_sl),
                                 as_stream(stream)});
}

int ssd_chunk_scan_bwd_dstates(const void* C, int64_t c_sb, int64_t c_sl, int64_t c_sg, const void* dout,
                               int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dA_cumsum,
                               void* dprev_states, int states_dtype, int64_t batch, int64_t seqlen,
                               int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                               const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(dout, d_sb, d_sl, d_sh, dtype, hdim));
  SSD_TRY(check_vec(C, c_sb, c_sl, c_sg, dtype, dstate));
  if (!dA_cumsum) return SSD_ERR_NULL;
  SSD_TRY(check_state(dprev_states, states_dtype, dtype));
  return dispatch_tpn(dtype, hdim, dstate,
                      StateLaunch<1>{dout, C, Strides3{d_sb, d_sl, d_sh}, Strides3{c_sb, c_sl, c_sg}, dA_cumsum,
                                     dA_cumsum, dprev_states, states_dtype, d, as_seq(seq_idx, seq_sb, seq_sl),
                                     as_stream(stream)});
}

size_t ssd_state_passing_bwd_workspace_bytes(int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim) {
  if (batch <= 0 || nchunks <= 0 || nheads <= 0 || dim <= 0) return 0;
  const int64_t tiles = (dim + 1023) / 1024;
  return (size_t)(batch * nheads * nchunks * tiles * 4) * sizeof(float);
}

int ssd_state_passing_bwd(const void* states, int states_dtype, const float* dA_chunk, int64_t da_sb, int64_t da_sh,
                          int64_t da_sc, const void* dout, int dout_dtype, const float* dfinal, void* dstates,
                          int dstates_dtype,
                          float* ddA_chunk, float* dinit, void* workspace, size_t workspace_bytes,
                          int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim, const int32_t* seq_idx,
                          int64_t seq_sb, int64_t seq_sl, int64_t seqlen, int64_t chunk, void* stream) {
  if (batch <= 0 || nchunks <= 0 || nheads <= 0 || dim <= 0) return SSD_ERR_SHAPE;
  if (dim % 4) return SSD_ERR_ALIGN;
  if (!dA_chunk || !ddA_chunk) return SSD_ERR_NULL;
  SSD_TRY(check_seq_chunks(seq_idx, seqlen, chunk, nchunks));
  const SeqIdx seq = as_seq(seq_idx, seq_sb, seq_sl);
  SSD_TRY(check_dtype(states_dtype));
  SSD_TRY(check_dtype(dout_dtype));
  SSD_TRY(check_dtype(dstates_dtype));
  SSD_TRY(check_f32(states));
  SSD_TRY(check_f32(dout));
  SSD_TRY(check_f32(dstates));
  SSD_TRY(check_f32(workspace));
  if (dfinal) SSD_TRY(check_f32(dfinal));
  if (dinit) SSD_TRY(check_f32(dinit));
  if (workspace_bytes < ssd_state_passing_bwd_workspace_bytes(batch, nchunks, nheads, dim)) return SSD_ERR_SHAPE;
  // eight elements per thread when every state-sized tensor is bfloat16 (16-byte accesses)
  const bool wide = states_dtype == SSD_BF16 && dout_dtype == SSD_BF16 && dstates_dtype == SSD_BF16 && dim % 8 == 0;
  const int per_block = wide ? 2048 : 1024;
  const int tiles = (int)((dim + per_block - 1) / per_block);
  const int64_t grid = batch * nheads * tiles;
  if (grid > 0x7fffffff || dim > (1 << 24)) return SSD_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  float* part = static_cast<float*>(workspace);
  // the three tensors are float32 or bfloat16 independently of each other
  auto launch = [&](auto ts, auto td, auto tg) {
    using TS = decltype(ts);
    using TD = decltype(td);
    using TG = decltype(tg);
    hipLaunchKernelGGL((ssd_state_passing_bwd_kernel<TS, TD, TG, 4>), dim3((unsigned)grid), dim3(256), 0, st,
                       (const TS*)states, dA_chunk, da_sb, da_sh, da_sc, (const TD*)dout, dfinal, (TG*)dstates, part,
                       dinit, (int)nheads, (int)nchunks, (int)dim, tiles, seq, (int)seqlen, (int)chunk);
  };
  auto pick_g = [&](auto ts, auto td) {
    if (dstates_dtype == SSD_BF16) launch(ts, td, bf16_t());
    else launch(ts, td, float());
  };
  auto pick_d = [&](auto ts) {
    if (dout_dtype == SSD_BF16) pick_g(ts, bf16_t());
    else pick_g(ts, float());
  };
  if (wide)
    hipLaunchKernelGGL((ssd_state_passing_bwd_kernel<bf16_t, bf16_t, bf16_t, 8>), dim3((unsigned)grid), dim3(256), 0,
                       st, (const bf16_t*)states, dA_chunk, da_sb, da_sh, da_sc, (const bf16_t*)dout, dfinal,
                       (bf16_t*)dstates, part, dinit, (int)nheads, (int)nchunks, (int)dim, tiles, seq, (int)seqlen,
                       (int)chunk);
  else if (states_dtype == SSD_BF16) pick_d(bf16_t());
  else pick_d(float());
  SSD_TRY(launched());
  const int64_t total = batch * nheads * nchunks;
  hipLaunchKernelGGL(ssd_state_passing_bwd_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     part, dA_chunk, da_sb, da_sh, da_sc, ddA_chunk, (int)nheads, (int)nchunks, tiles * 4,
                     dinit ? 1 : 0, total, seq, (int)seqlen, (int)chunk);
  return launched();
}

size_t ssd_chunk_scan_state_passing_bwd_workspace_bytes(int64_t batch, int64_t nchunks, int64_t nheads) {
  if (batch <= 0 || nchunks <= 0 || nheads <= 0) return 0;
  return (size_t)(batch * nheads * nchunks * 8) * sizeof(float);  // a partial dot per wave
}

int ssd_chunk_scan_state_passing_bwd(const void* C, int64_t c_sb, int64_t c_sl, int64_t c_sg, const void* dout,
                                     int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dA_cumsum,
                                     const void* states, int states_dtype, const float* dfinal, void* dstates,
                                     int dstates_dtype, float* ddA_chunk, float* dinit, void* workspace,
                                     size_t workspace_bytes, int64_t batch, int64_t seqlen, int64_t nheads,
                                     int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  SSD_TRY(check_dtype(states_dtype));
  SSD_TRY(check_dtype(dstates_dtype));
  // what the kernel is written for: its tiles and its three state buffers in LDS have these sizes
  if (dtype != SSD_BF16 || states_dtype != SSD_BF16 || hdim != 64 || dstate != 128 || chunk % 64 || chunk < 128)
    return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(dout, d_sb, d_sl, d_sh, dtype, hdim));
  SSD_TRY(check_vec(C, c_sb, c_sl, c_sg, dtype, dstate));
  SSD_TRY(check_f32(dA_cumsum));  // fetched in 16-byte pieces
  SSD_TRY(check_f32(states));
  SSD_TRY(check_f32(dstates));
  SSD_TRY(check_f32(workspace));
  if (!ddA_chunk) return SSD_ERR_NULL;
  if (dfinal) SSD_TRY(check_f32(dfinal));
  if (dinit) SSD_TRY(check_f32(dinit));
  if (workspace_bytes < ssd_chunk_scan_state_passing_bwd_workspace_bytes(batch, d.C, nheads)) return SSD_ERR_SHAPE;
  const Strides3 sd{d_sb, d_sl, d_sh}, sc{c_sb, c_sl, c_sg};
  // (the kernel keeps the byte offset of a row inside a stage in 32 bits)
  if (!forward_strides(sd) || !forward_strides(sc) || sd.sl >= (int64_t(1) << 24) || sc.sl >= (int64_t(1) << 24))
    return SSD_ERR_UNSUPPORTED;
  if (batch * nheads > 0x7fffffff) return SSD_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  float* part = static_cast<float*>(workspace);
  constexpr int smem = WalkBwdDmaSmem::kBytes;
  auto launch = [&](auto tg) -> int {
    using TG = decltype(tg);
    auto kernel = ssd_state_walk_bwd_dma_kernel<TG>;
    SSD_TRY(allow_smem(kernel, smem));
    hipLaunchKernelGGL(kernel, dim3((unsigned)(batch * nheads)), dim3(512), smem, st, (const bf16_t*)dout, sd,
                       (const bf16_t*)C, sc, dA_cumsum, (const bf16_t*)states, dfinal, (TG*)dstates, part, dinit,
                       (int)nheads, (int)(nheads / ngroups), (int)seqlen, (int)chunk, (int)d.C);
    return launched();
  };
  SSD_TRY(dstates_dtype == SSD_BF16 ? launch(bf16_t()) : launch(float()));
  // ddA_chunk[b,h,c] = exp(dA_cumsum[b,h,c,chunk-1]) * the sum of the eight partial dots
  const int64_t total = batch * nheads * d.C;
  hipLaunchKernelGGL(ssd_state_passing_bwd_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     part, dA_cumsum + (chunk - 1), nheads * d.C * chunk, d.C * chunk, chunk, ddA_chunk, (int)nheads,
                     (int)d.C, 8, dinit ? 1 : 0, total, as_seq(nullptr, 0, 0), (int)seqlen, (int)chunk);
  return launched();
}

int ssd_chunk_state_bwd_db(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                           const float* dt, const float* dA_cumsum, const void* dstates, int states_dtype,
                           const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, float* dB, float* ddA_cumsum,
                           int64_t batch, int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim,
                           int64_t dstate, int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl,
                           void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  if (!dB) return SSD_ERR_NULL;
  SSD_TRY(check_f32(dt));  // fetched in 16-byte pieces
  SSD_TRY(check_f32(dA_cumsum));
  SSD_TRY(check_state(dstates, states_dtype, dtype));
  if (B && !ddA_cumsum) return SSD_ERR_NULL;
  if (B) SSD_TRY(check_vec(B, b_sb, b_sl, b_sg, dtype, dstate));
  hipStream_t st = as_stream(stream);
  SSD_TRY(dispatch_tpn(dtype, hdim, dstate,
                       GroupLaunch<0>{x, Strides3{x_sb, x_sl, x_sh}, dstates, states_dtype, dt, dA_cumsum, B,
                                      Strides3{b_sb, b_sl, b_sg}, dB, ddA_cumsum, d,
                                      as_seq(seq_idx, seq_sb, seq_sl), st}));
  if (!B) return SSD_OK;
  return launch_row_cumsum(ddA_cumsum, chunk, batch * nheads * d.C, st);
}

int ssd_chunk_scan_bwd_dc(const void* dout, int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype,
                          const float* dA_cumsum, const void* prev_states, int states_dtype, const void* C,
                          int64_t c_sb,
                          int64_t c_sl, int64_t c_sg, float* dC, float* ddA_cumsum_prev, int64_t batch,
                          int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate,
                          int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  SSD_TRY(check_vec(dout, d_sb, d_sl, d_sh, dtype, hdim));
  if (!dC) return SSD_ERR_NULL;
  SSD_TRY(check_f32(dA_cumsum));  // fetched in 16-byte pieces
  SSD_TRY(check_state(prev_states, states_dtype, dtype));
  if (C && !ddA_cumsum_prev) return SSD_ERR_NULL;
  if (C) SSD_TRY(check_vec(C, c_sb, c_sl, c_sg, dtype, dstate));
  return dispatch_tpn(dtype, hdim, dstate,
                      GroupLaunch<1>{dout, Strides3{d_sb, d_sl, d_sh}, prev_states, states_dtype, dA_cumsum, dA_cumsum,
                                     C,
                                     Strides3{c_sb, c_sl, c_sg}, dC, ddA_cumsum_prev, d,
                                     as_seq(seq_idx, seq_sb, seq_sl), as_stream(stream)});
}

int ssd_chunk_scan_chunk_state_bwd_dx(const float* cb, const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                                      const void* dout, int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype,
                                      const float* dt, const float* dA_cumsum, const void* B, int64_t b_sb,
                                      int64_t b_sl, int64_t b_sg, const void* dstates, int states_dtype, const float* D,
                                      int d_has_hdim, void* dx, int64_t dx_sb, int64_t dx_sl, int64_t dx_sh,
                                      float* ddt, int64_t batch, int64_t seqlen, int64_t nheads,
                                      int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                                      const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, float* dD_partial,
                                      void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (!dim_ok(hdim) || !dim_ok(dstate)) return SSD_ERR_UNSUPPORTED;
  if (dD_partial && !D) return SSD_ERR_NULL;
  if (dD_partial) SSD_TRY(check_f32(dD_partial));
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  SSD_TRY(check_vec(dout, d_sb, d_sl, d_sh, dtype, hdim));
  SSD_TRY(check_vec(dx, dx_sb, dx_sl, dx_sh, dtype, hdim));
  SSD_TRY(check_vec(B, b_sb, b_sl, b_sg, dtype, dstate));
  if (!dt || !dA_cumsum || !ddt) return SSD_ERR_NULL;
  SSD_TRY(check_f32(cb));
  SSD_TRY(check_state(dstates, states_dtype, dtype));
  if (batch * d.C * nheads * ((chunk + 63) / 64) > 0x7fffffff) return SSD_ERR_SHAPE;
  return dispatch_tpn(dtype, hdim, dstate,
                      DxLaunch{cb, x, dout, B, Strides3{x_sb, x_sl, x_sh}, Strides3{d_sb, d_sl, d_sh},
                               Strides3{b_sb, b_sl, b_sg}, Strides3{dx_sb, dx_sl, dx_sh}, dt, dA_cumsum, dstates,
                               states_dtype, D,
                               d_has_hdim, dx, ddt, d, as_seq(seq_idx, seq_sb, seq_sl), dD_partial,
                               as_stream(stream)});
}

int64_t ssd_chunk_scan_chunk_state_bwd_dx_dD_slots(int dtype, int64_t hdim, int64_t dstate, int64_t chunk) {
  if (check_dtype(dtype) != SSD_OK || !dim_ok(hdim) || !dim_ok(dstate)) return 0;
  if (chunk <= 0 || chunk > 1024 || chunk % 4) return 0;
  return dispatch_tpn(dtype, hdim, dstate, DxSlots{chunk});
}

static size_t ddAcs_part_floats(const Dims& d) {
  const int64_t MT = (d.Q + ema::kBM - 1) / ema::kBM;
  return (size_t)(d.batch * d.nh * d.C * MT * d.Q);
}

size_t ssd_chunk_scan_bwd_ddAcs_workspace_bytes(int64_t batch, int64_t seqlen, int64_t nheads, int64_t chunk) {
  Dims d;
  if (check_dims(batch, seqlen, nheads, 1, 0, 0, chunk, &d) != SSD_OK) return 0;
  return (ddAcs_part_floats(d) + (size_t)(batch * nheads * d.C * chunk)) * sizeof(float);
}

int ssd_chunk_scan_bwd_ddAcs(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, const void* dout,
                             int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dt,
                             const float* dA_cumsum, const float* cb, float* ddA_cumsum, void* workspace,
                             size_t workspace_bytes, int64_t batch, int64_t seqlen, int64_t nheads,
                             int64_t ngroups, int64_t hdim, int64_t chunk, void* stream) {
  Dims d;
  SSD_TRY(check_dims(batch, seqlen, nheads, ngroups, hdim, 0, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (hdim <= 0 || hdim > (1 << 16)) return SSD_ERR_SHAPE;
  SSD_TRY(check_vec(x, x_sb, x_sl, x_sh, dtype, hdim));
  SSD_TRY(check_vec(dout, d_sb, d_sl, d_sh, dtype, hdim));
  if (!dt || !dA_cumsum || !cb || !ddA_cumsum) return SSD_ERR_NULL;
  SSD_TRY(check_f32(workspace));
  if (workspace_bytes < ssd_chunk_scan_bwd_ddAcs_workspace_bytes(batch, seqlen, nheads, chunk)) return SSD_ERR_SHAPE;
  hipStream_t st = as_stream(stream);
  if ((chunk == 64 || chunk == 128 || chunk == 256) && dim_ok(hdim)) {
    // one workgroup per (b, c, h) does everything, prefix sum included
    const int64_t wgs = batch * nheads * d.C;
    if (wgs > 0x7fffffff) return SSD_ERR_SHAPE;
    const Strides3 sx{x_sb, x_sl, x_sh}, sd{d_sb, d_sl, d_sh};
    const int hpg = (int)(nheads / ngroups);
#define SSD_DDA_LAUNCH(T, P)                                                                                    \
  do {                                                                                                          \
    auto kernel = ssd_ddA_causal_kernel<T, P>;                                                                  \
    constexpr int smem = DdaSmem<T, P>::kBytes;                                                                 \
    SSD_TRY(allow_smem(kernel, smem));                                                                          \
    hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(256), smem, st, (const T*)x, sx, (const T*)dout, sd,  \
                       dt, dA_cumsum, cb, ddA_cumsum, (int)nheads, hpg, (int)ngroups, (int)seqlen, (int)chunk,  \
                       (int)d.C);                                                                               \
  } while (0)
    if (dtype == SSD_BF16) {
      if (hdim == 64) SSD_DDA_LAUNCH(bf16_t, 64);
      else SSD_DDA_LAUNCH(bf16_t, 128);
    } else {
      if (hdim == 64) SSD_DDA_LAUNCH(float, 64);
      else SSD_DDA_LAUNCH(float, 128);
    }
#undef SSD_DDA_LAUNCH
    return launched();
  }
  float* part = static_cast<float*>(workspace);
  float* rowsum = part + ddAcs_part_floats(d);
  const int MT = (int)((d.Q + ema::kBM - 1) / ema::kBM);
  const int64_t grid = batch * nheads * d.C * MT;
  if (grid > 0x7fffffff) return SSD_ERR_SHAPE;
  const ema::SeqStrides sx{x_sb, x_sl, x_sh}, sd{d_sb, d_sl, d_sh};
  const int hpg = (int)(nheads / ngroups);
  if (dtype == SSD_BF16)
    hipLaunchKernelGGL((ema::da_gemm_kernel<bf16_t>), dim3((unsigned)grid), dim3(256), 0, st, (const bf16_t*)x, sx,
                       (const bf16_t*)dout, sd, dA_cumsum, part, rowsum, (int)nheads, (int)seqlen, (int)hdim,
                       (int)chunk, (int)d.C, MT, dt, cb, hpg, (int)ngroups);
  else
    hipLaunchKernelGGL((ema::da_gemm_kernel<float>), dim3((unsigned)grid), dim3(256), 0, st, (const float*)x, sx,
                       (const float*)dout, sd, dA_cumsum, part, rowsum, (int)nheads, (int)seqlen, (int)hdim,
                       (int)chunk, (int)d.C, MT, dt, cb, hpg, (int)ngroups);
  SSD_TRY(launched());
  const int64_t total = batch * nheads * d.C;
  hipLaunchKernelGGL(ema::da_finish_kernel<ema::kBM>, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, st, part,
                     rowsum, ddA_cumsum, (int)chunk, MT, total);
  return launched();
}

int ssd_chunk_state_varlen(const void* B, int64_t b_sl, int64_t b_sg, const void* x, int64_t x_sl, int64_t x_sh,
                           int dtype, const float* dt, const float* dA_cumsum, const void* chunk_states,
                           int states_dtype, const int32_t* cu_seqlens, float* states, int64_t nseq, int64_t seqlen, int64_t nheads,
                           int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream) {
  Dims d;
  SSD_TRY(check_dims(1, seqlen, nheads, ngroups, hdim, dstate, chunk, &d));
  SSD_TRY(check_dtype(dtype));
  if (nseq <= 0 || nseq > 65535 || hdim <= 0 || dstate <= 0 || hdim > 4096 || dstate > 4096) return SSD_ERR_SHAPE;
  if (states_dtype != SSD_F32 && states_dtype != dtype) return SSD_ERR_DTYPE;
  if (!B || !x || !dt || !dA_cumsum || !chunk_states || !cu_seqlens || !states) return SSD_ERR_NULL;
  const int64_t tiles = ((hdim + 63) / 64) * ((dstate + 63) / 64);
  const dim3 grid((unsigned)tiles, (unsigned)nseq, (unsigned)nheads);
  const int hpg = (int)(nheads / ngroups);
  if (dtype == SSD_BF16 && states_dtype == SSD_BF16)
    hipLaunchKernelGGL((ssd_chunk_state_varlen_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, as_stream(stream),
                       (const bf16_t*)x, x_sl, x_sh, (const bf16_t*)B, b_sl, b_sg, dt, dA_cumsum,
                       (const bf16_t*)chunk_states, cu_seqlens, states, (int)seqlen, (int)nheads, hpg, (int)hdim,
                       (int)dstate, (int)chunk, (int)d.C);
  else if (dtype == SSD_BF16)
    hipLaunchKernelGGL((ssd_chunk_state_varlen_kernel<bf16_t, float>), grid, dim3(256), 0, as_stream(stream),
                       (const bf16_t*)x, x_sl, x_sh, (const bf16_t*)B, b_sl, b_sg, dt, dA_cumsum,
                       (const float*)chunk_states, cu_seqlens, states, (int)seqlen, (int)nheads, hpg, (int)hdim,
                       (int)dstate, (int)chunk, (int)d.C);
  else
    hipLaunchKernelGGL((ssd_chunk_state_varlen_kernel<float, float>), grid, dim3(256), 0, as_stream(stream),
                       (const float*)x, x_sl, x_sh, (const float*)B, b_sl, b_sg, dt, dA_cumsum,
                       (const float*)chunk_states, cu_seqlens, states, (int)seqlen, (int)nheads, hpg, (int)hdim,
                       (int)dstate, (int)chunk, (int)d.C);
  return launched();
}

#ifdef SSD_TIMING
// Development aid, only in builds with -DSSD_TIMING: installs the per-workgroup timestamp buffer.
int ssd_debug_set_timing(void* buf) {
  return hipMemcpyToSymbol(HIP_SYMBOL(ssd::g_ssd_timing), &buf, sizeof(buf)) == hipSuccess ? 0 : -6;
}
#endif

}  // extern "C"
