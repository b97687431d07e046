// Forward kernels of the Mamba-2 SSD chunked scan (gfx950, wave64).
//
// Five stages, one kernel each, with the tensor layouts of the reference's launchers in
// kernels/mamba_kernels/:
//   chunk_cumsum   dt -> processed dt and the per-chunk cumsum of dt * A        (DPP scan)
//   chunk_state    states[p][n] = sum_k x[k][p] * (B[k][n] * w_k)               (MFMA)
//   state_passing  the inter-chunk recurrence over (hdim x dstate) states       (HBM stream)
//   bmm_chunk      CB[m][k] = sum_n C[m][n] * B[k][n]                           (MFMA)
//   chunk_scan     out = exp(dA_m) * C.prev + (CB o decay o dt, causal) x + D x (MFMA)
//
// MFMA operands are staged in LDS.  A tile that is contracted along its rows (x[k][p],
// B[k][n]) is read with the transposing LDS read for bf16 (four scalar reads for f32); a tile
// contracted along its columns (C[m][n], prev[p][n], the weighted CB[m][k]) is read with one
// 16-byte LDS read per lane.  Accumulation is float32 throughout; operands that the reference
// rounds to the input type before its dot (the weighted B, the weighted CB, prev) are rounded
// the same way here.
#pragma once
#include <type_traits>

#include "ema_device.h"

namespace ssd {

using ema::acc_row;
using ema::bf16_t;
using ema::floatx16;
using ema::load16;
using ema::load16_stream;
using ema::mma_group;
using ema::store16;
using ema::store16_stream;
using ema::Vec16;
using ema::wave_inclusive_scan;

#ifdef SSD_TIMING
// Development aid: per-workgroup phase timestamps into a global buffer (never built into the library).
__device__ long long* g_ssd_timing = nullptr;
#define SSD_TSTAMP(slot)                                                                              \
  do {                                                                                                \
    if (threadIdx.x == 0 && g_ssd_timing) g_ssd_timing[(int64_t)blockIdx.x * 8 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define SSD_TSTAMP(slot) \
  do {                   \
  } while (0)
#endif

// Element strides of a (batch, position, head-or-group) tensor whose last axis is dense.
struct Strides3 {
  int64_t sb, sl, sh;
};

// Sequence ids of a packed batch: (batch, seqlen) int32 addressed by element strides; p is null
// when the batch is not packed.  Positions with different ids belong to different sequences and
// do not see each other's state.
struct SeqIdx {
  const int* p;
  int64_t sb, sl;
};

// The ids of one chunk.  at(-1) is the last position of the previous chunk.
struct ChunkSeq {
  const int* p;
  int64_t sl;
  __device__ __forceinline__ bool on() const { return p != nullptr; }
  __device__ __forceinline__ int at(int k) const { return p[(int64_t)k * sl]; }
  // id that the state entering chunk c carries: the reference starts from id 0
  __device__ __forceinline__ int entering(int c) const { return c > 0 ? at(-1) : 0; }
};
__device__ __forceinline__ ChunkSeq chunk_seq(SeqIdx s, int64_t b, int c, int Q) {
  return ChunkSeq{s.p ? s.p + b * s.sb + (int64_t)c * Q * s.sl : nullptr, s.sl};
}
// Whether the state survives chunk c: the id at the end of the chunk equals the id at the end of
// the previous one (0 before the first chunk).
__device__ __forceinline__ bool chunk_keeps_state(SeqIdx s, int64_t b, int c, int Q, int L) {
  if (!s.p) return true;
  const int* q = s.p + b * s.sb;
  const int cur = q[(int64_t)(min((c + 1) * Q, L) - 1) * s.sl];
  const int before = c > 0 ? q[(int64_t)(c * Q - 1) * s.sl] : 0;
  return cur == before;
}

// Workgroups are dealt to the 8 XCDs round-robin by their index, and each XCD has its own L2.
// This maps the hardware index to a logical one whose consecutive values run on the same XCD,
// so that workgroups which share operands (the heads of a group, the row tiles of a chunk) find
// them in that L2 instead of fetching them once per XCD.  A bijection on [0, nblocks).
__device__ __forceinline__ int xcd_local_index(int bid, int nblocks) {
  constexpr int kXcds = 8;
  const int per = nblocks / kXcds;
  if (bid >= per * kXcds) return bid;  // the tail that does not fill a round keeps its place
  return (bid % kXcds) * per + bid / kXcds;
}

// ------------------------------------------------------------------ operand fragments
// Both return, for lane l, EPL = Vec16<T>::N consecutive contraction indices starting at
// k0 + EPL * (l / 32), for row or column (l % 32) of the 32-wide block: the register layout
// mma_group expects for either operand.

// tile[row][k], contracted along k (row-major)
template <typename T>
__device__ __forceinline__ Vec16<T> frag_rows(const T* tile, int pitch, int row0, int k0, int lane) {
  return load16(tile + (row0 + (lane & 31)) * pitch + k0 + Vec16<T>::N * (lane >> 5));
}

// tile[k][col], contracted along k (k-major)
__device__ __forceinline__ Vec16<bf16_t> frag_cols(const bf16_t* tile, int pitch, int k0, int col0,
                                                   int lane) {
  return ema::lds_read_kmajor(tile, pitch, k0, col0, lane);
}
__device__ __forceinline__ Vec16<float> frag_cols(const float* tile, int pitch, int k0, int col0,
                                                  int lane) {
  const float* p = tile + (k0 + 4 * (lane >> 5)) * pitch + col0 + (lane & 31);
  Vec16<float> r;
  r.raw = make_float4(p[0], p[pitch], p[2 * pitch], p[3 * pitch]);
  return r;
}

template <typename T>
struct Tile {
  static constexpr int EPL = Vec16<T>::N;
  static constexpr int KG = 2 * EPL;  // contraction extent of one mma_group
  // LDS pitch (elements) of a tile with `cols` dense columns: 16 bytes of padding
  static constexpr int pitch(int cols) { return cols + EPL; }
  // LDS pitch of a tile that is contracted along its rows (read with frag_cols).  The LDS has 64
  // banks of 4 bytes.  One transposing read takes, per half wave, 64 adjacent bytes of four
  // consecutive rows: with 64 bytes of padding (bf16 rows are multiples of 128 bytes here) the
  // four rows fall into four different quarters of the 256-byte bank period.  The float32 form
  // reads 128 adjacent bytes of two rows four apart per instruction: 32 bytes of padding put them
  // into different halves.
  static constexpr int kpitch(int cols) { return cols + (sizeof(T) == 2 ? 32 : 8); }
};

// ------------------------------------------------------------------ copies from global memory into LDS
// The load unit can write what it fetches straight into LDS, without passing through registers:
// such copies occupy no registers while they are under way, so how many a workgroup has in flight is
// bounded by LDS alone.  They count as vector-memory loads of the requesting wave and complete in
// order with its other loads and stores.
typedef __attribute__((address_space(3))) void lds_void_t;

// 64 lanes x 16 bytes from global memory into LDS: lane l's piece, at base + lane_offset bytes, lands at
// lds_base + 16 * l.  base and lds_base are the same for the whole wave (scalar registers), so a loop that only
// moves the base spends no vector instructions on addresses.  Written as assembly so that the compiler does
// not make every later LDS read wait for all copies under way (given the builtin it does, whatever the
// addresses); the caller waits for the counter (s_waitcnt vmcnt) and passes a barrier before another wave
// reads the data.  m0, which carries the LDS address, is put back, so the compiler need not know that it
// changes; five wait states precede the load because its scalar base may just have been written by vector
// instructions (v_readfirstlane), which the compiler cannot see from outside the assembly.
__device__ __forceinline__ void copy16_to_lds(const void* base, unsigned lane_offset, void* lds_base) {
  const unsigned lds = (unsigned)(uintptr_t)(lds_void_t*)lds_base;
  const uint64_t wide = reinterpret_cast<uint64_t>(base);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(wide >> 32));
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)wide);  // (unsigned: no sign extension below)
  base = reinterpret_cast<const void*>(((uint64_t)hi << 32) | (uint64_t)lo);
  unsigned keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
               : "=&s"(keep)
               : "v"(lane_offset), "s"(base), "s"(lds)
               : "memory");
}

__device__ __forceinline__ void zero_acc(floatx16& a) {
#pragma unroll
  for (int v = 0; v < 16; ++v) a[v] = 0.f;
}

// Rows [row0, row0 + ROWS) x COLS dense columns of a global tensor into an LDS tile, 16 bytes
// per thread and step; rows at or past `limit` read as zero.  A `scale` other than NoScale
// multiplies row r by scale(r) in float32 before the value is rounded to T.
struct NoScale {
  __device__ __forceinline__ float operator()(int) const { return 1.f; }
};

// STREAM: the rows are read with the non-temporal hint (data of one head that no other workgroup
// is about to read through the same L2).
template <typename T, int ROWS, int COLS, typename F, bool STREAM = false>
__device__ __forceinline__ void stage_rows(T* tile, const T* __restrict__ g, int64_t row_stride, int row0,
                                           int limit, int tid, F scale) {
  constexpr int EPL = Vec16<T>::N, VPR = COLS / EPL, P = Tile<T>::pitch(COLS);
  static_assert((ROWS * VPR) % 256 == 0, "tile must split evenly over 256 threads");
  constexpr int CNT = ROWS * VPR / 256, GRP = CNT < 8 ? CNT : 8;
  static_assert(CNT % GRP == 0, "load groups must divide the tile");
  // Up to eight loads go out before the first LDS store of a group (the compiler otherwise tends
  // to wait for each load in turn to save registers).  They are unconditional, from rows clamped
  // into the sequence (limit >= 1): a load inside a branch would have to complete before the
  // next one is issued.
#pragma unroll
  for (int i0 = 0; i0 < CNT; i0 += GRP) {
    Vec16<T> v[GRP];
#pragma unroll
    for (int i = 0; i < GRP; ++i) {
      const int idx = tid + 256 * (i0 + i);
      const int r = idx / VPR, cv = (idx % VPR) * EPL;
      const int row = row0 + r < limit ? row0 + r : limit - 1;
      v[i] = STREAM ? load16_stream(g + (int64_t)row * row_stride + cv) : load16(g + (int64_t)row * row_stride + cv);
    }
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < GRP; ++i) {
      const int idx = tid + 256 * (i0 + i);
      const int r = idx / VPR, cv = (idx % VPR) * EPL;
      const bool in = row0 + r < limit;
      if constexpr (!std::is_same<F, NoScale>::value) {
        const float s = scale(in ? row0 + r : limit - 1);
        float t[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) t[e] = v[i].get(e) * s;
        v[i].set_all(t);
      }
      if (!in) v[i].zero();
      store16(tile + r * P + cv, v[i]);
    }
  }
}
// The two halves of stage_rows for tiles of at most eight 16-byte pieces per thread: the loads
// (into registers) and, later, the scaling, masking and LDS stores.  A kernel that has the next
// tile's loads in flight while it works on the current one calls them apart.  Up to two float32
// values per row (aux0[row], aux1[row]; null = not wanted) travel with the pieces, so that a
// row scale computed from them costs no load at store time.
template <typename T, int ROWS, int COLS, int PITCH = Tile<T>::pitch(COLS)>
struct RowPieces {
  static constexpr int EPL = Vec16<T>::N, VPR = COLS / EPL, CNT = ROWS * VPR / 256;
  static_assert((ROWS * VPR) % 256 == 0 && CNT <= 8, "tile must split evenly over 256 threads");
  Vec16<T> v[CNT];
  float a0[CNT], a1[CNT];
  // BOTH: aux0 and aux1 are given (no test of the pointers between the loads)
  template <bool STREAM = false, bool BOTH = false>
  __device__ __forceinline__ void load(const T* __restrict__ g, int64_t row_stride, int row0, int limit, int tid,
                                       const float* __restrict__ aux0 = nullptr,
                                       const float* __restrict__ aux1 = nullptr) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int idx = tid + 256 * i;
      const int row = min(row0 + idx / VPR, limit - 1);
      const T* src = g + (int64_t)row * row_stride + (idx % VPR) * EPL;
      v[i] = STREAM ? load16_stream(src) : load16(src);
      if (BOTH || aux0) a0[i] = aux0[row];
      if (BOTH || aux1) a1[i] = aux1[row];
    }
  }
  // scale(row, aux0[row], aux1[row]) multiplies the row; NoScale leaves it
  template <typename F>
  __device__ __forceinline__ void store(T* tile, int row0, int limit, int tid, F scale) {
    constexpr int P = PITCH;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / VPR, cv = (idx % VPR) * EPL;
      const bool in = row0 + r < limit;
      if constexpr (!std::is_same<F, NoScale>::value) {
        const float s = scale(in ? row0 + r : limit - 1, a0[i], a1[i]);
        float t[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) t[e] = v[i].get(e) * s;
        v[i].set_all(t);
      }
      if (!in) v[i].zero();
      store16(tile + r * P + cv, v[i]);
    }
  }
};

// ------------------------------------------------------------------------------------
// chunk_cumsum.  One workgroup per (b, c, group of HT heads), HT a power of two up to 8.  dt is
// (batch, seqlen, nheads) with the heads innermost, so the workgroup reads its Q x HT tile with the
// heads across adjacent lanes, processes it (bias, softplus with the identity above 20, clamp; 0
// past the sequence) and transposes it through LDS; then one wave per head scans dA = dt * A[h]
// across the chunk with DPP, each lane owning ceil(Q/64) consecutive positions.  Outputs are
// (b, nh, C, Q) float32.  LDS: HT * (Q + 1) floats.
// ------------------------------------------------------------------------------------
template <typename TD>
__global__ __launch_bounds__(256) void ssd_cumsum_kernel(const TD* __restrict__ dt, Strides3 sd,
                                                         const float* __restrict__ A,
                                                         const float* __restrict__ dt_bias,
                                                         float* __restrict__ dA_cs, float* __restrict__ dt_out,
                                                         int nh, int L, int Q, int C, int softplus,
                                                         float dt_min, float dt_max, int HT, int hgroups) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* tile = reinterpret_cast<float*>(smem);  // [HT][Q + 1]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);  // a chunk's head groups share lines of dt
  const int hg = bid % hgroups;
  const int c = (bid / hgroups) % C;
  const int64_t b = bid / (hgroups * C);
  const int h0 = hg * HT;
  const int limit = min(Q, L - c * Q);
  const int pitch = Q + 1;
  {
    const int j = tid % HT, qstep = 256 / HT;
    const int h = min(h0 + j, nh - 1);
    const TD* src = dt + b * sd.sb + (int64_t)c * Q * sd.sl + (int64_t)h * sd.sh;
    const float bias = dt_bias ? dt_bias[h] : 0.f;
    constexpr int U = 8;  // loads in flight per thread
    for (int qb = tid / HT; qb < Q; qb += U * qstep) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = (float)src[(int64_t)min(qb + u * qstep, limit - 1) * sd.sl];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int q = qb + u * qstep;
        float t = v[u] + bias;
        if (softplus && t <= 20.f) t = log1pf(__expf(t));
        t = fminf(fmaxf(t, dt_min), dt_max);
        if (q < Q) tile[j * pitch + q] = q < limit ? t : 0.f;
      }
    }
  }
  __syncthreads();
  const int per = (Q + 63) >> 6;
  const int q0 = lane * per;
  for (int jj = wave; jj < HT && h0 + jj < nh; jj += 4) {
    const int h = h0 + jj;
    const float a = A[h];
    const float* row = tile + jj * pitch;
    float local = 0.f;
    for (int i = 0; i < per; ++i)
      if (q0 + i < Q) local += row[q0 + i] * a;
    float run = wave_inclusive_scan(local) - local;
    const int64_t id = (b * nh + h) * C + c;
    float* o_cs = dA_cs + id * Q;
    float* o_dt = dt_out + id * Q;
    if (per == 4 && Q == 256) {  // the lane's four positions leave as one 16-byte store per output
      float4 v4, c4;
      v4.x = row[q0], v4.y = row[q0 + 1], v4.z = row[q0 + 2], v4.w = row[q0 + 3];
      c4.x = run += v4.x * a;
      c4.y = run += v4.y * a;
      c4.z = run += v4.z * a;
      c4.w = run += v4.w * a;
      *reinterpret_cast<float4*>(o_dt + q0) = v4;
      *reinterpret_cast<float4*>(o_cs + q0) = c4;
      continue;
    }
    for (int i = 0; i < per; ++i) {
      const int q = q0 + i;
      if (q < Q) {
        const float v = row[q];
        run += v * a;
        o_dt[q] = v;
        o_cs[q] = run;
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// chunk_state (MODE 0) and its mirror image in the backward, dstates (MODE 1).  One workgroup
// (4 waves) per (b, c, h):
//   MODE 0  states[p][n] = sum_k x[k][p] * round_T(B[k][n] * exp(min(dA_last - dA_k, 0)) * dt_k)
//   MODE 1  dprev[p][n]  = sum_k round_T(dout[k][p] * exp(dA_k)) * C[k][n]
// (x / B stand for dout / C in MODE 1; dt is not read).  In a packed batch position k only
// counts if its id equals the id of the chunk's last position (MODE 0; none counts if that id is
// negative) or of the previous chunk's last position (MODE 1).  The chunk is walked in stages of 64
// rows; both operands are contracted along their rows.  The (P/32) x (N/32) output blocks are
// dealt to the waves round-robin.
// ------------------------------------------------------------------------------------
template <typename T, int P, int N>
struct StateSmem {
  static constexpr int KT = 64, PX = Tile<T>::kpitch(P), PB = Tile<T>::kpitch(N);
  static constexpr int kStage = KT * (PX + PB) * (int)sizeof(T);
  // One stage in LDS.  The next stage waits in registers while this one is multiplied, so a second
  // LDS buffer only saves a barrier per stage, and at 53 KB it allowed three workgroups per CU
  // where the registers allow four (hdim 64, dstate 128): one buffer measured 7 % faster.
  static constexpr int kBytes = kStage;
};

template <typename T, int P, int N, int MODE, typename TO>
__global__ __launch_bounds__(256) void ssd_chunk_state_kernel(
    const T* __restrict__ x, Strides3 sx, const T* __restrict__ B, Strides3 sB,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, TO* __restrict__ states, int nh,
    int heads_per_group, int L, int Q, int C, SeqIdx seq) {
  using S = StateSmem<T, P, N>;
  constexpr int KT = S::KT, PX = S::PX, PB = S::PB, KG = Tile<T>::KG;
  constexpr int MB = P / 32, NB = N / 32, BPW = MB * NB / 4;
  static_assert(MB * NB % 4 == 0, "output blocks must split over 4 waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* xs = reinterpret_cast<T*>(smem);
  T* bs = xs + KT * PX;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int h = bid % nh;
  const int c = (bid / nh) % C;
  const int64_t b = bid / (nh * C);
  const int limit = min(Q, L - c * Q);
  const float* dAp = dA_cs + ((b * nh + h) * C + c) * (int64_t)Q;
  const float* dtp = dt + ((b * nh + h) * C + c) * (int64_t)Q;
  const float dA_last = dAp[Q - 1];
  const T* xg = x + b * sx.sb + (int64_t)c * Q * sx.sl + h * sx.sh;
  const T* Bg = B + b * sB.sb + (int64_t)c * Q * sB.sl + (h / heads_per_group) * sB.sh;
  const ChunkSeq sq = chunk_seq(seq, b, c, Q);
  const int seq_ref = !sq.on() ? 0 : (MODE == 0 ? sq.at(limit - 1) : sq.entering(c));
  const bool seq_dead = MODE == 0 && seq_ref < 0;

  floatx16 acc[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) zero_acc(acc[i]);

  // Stage s + 1 is requested before the products of stage s and written to LDS after them: the
  // loads have the products to hide behind.
  auto scale_b = [&](int k, float dA_k, float dt_k) {
    const float w = __expf(fminf(dA_last - dA_k, 0.f)) * dt_k;
    return (sq.on() && (seq_dead || sq.at(k) != seq_ref)) ? 0.f : w;
  };
  auto scale_x = [&](int k, float dA_k, float) {
    const float w = __expf(dA_k);
    return (sq.on() && sq.at(k) != seq_ref) ? 0.f : w;
  };
  RowPieces<T, KT, P, PX> px;
  RowPieces<T, KT, N, PB> pb;
  auto request = [&](int k0) {  // the pieces of a stage and the per-row values their scale needs
    px.template load<true>(xg, sx.sl, k0, limit, tid, MODE == 1 ? dAp : nullptr);
    pb.load(Bg, sB.sl, k0, limit, tid, MODE == 0 ? dAp : nullptr, MODE == 0 ? dtp : nullptr);
  };
  request(0);
  T* xb = xs;
  T* bb = bs;
  for (int k0 = 0; k0 < limit; k0 += KT) {
    if (k0 > 0) __syncthreads();  // every wave is done with the stage that is overwritten now
    if (MODE == 0) {
      px.store(xb, k0, limit, tid, NoScale());
      pb.store(bb, k0, limit, tid, scale_b);
    } else {
      px.store(xb, k0, limit, tid, scale_x);
      pb.store(bb, k0, limit, tid, NoScale());
    }
    __syncthreads();
    if (k0 + KT < limit) request(k0 + KT);
#pragma unroll
    for (int kk = 0; kk < KT; kk += KG) {
#pragma unroll
      for (int i = 0; i < BPW; ++i) {
        const int j = wave + 4 * i, mi = j % MB, ni = j / MB;
        mma_group(frag_cols(xb, PX, kk, 32 * mi, lane), frag_cols(bb, PB, kk, 32 * ni, lane), acc[i]);
      }
    }
  }
  TO* out = states + (((b * C + c) * nh + h) * (int64_t)P) * N;
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int j = wave + 4 * i, mi = j % MB, ni = j / MB;
#pragma unroll
    for (int v = 0; v < 16; ++v)
      __builtin_nontemporal_store((TO)acc[i][v], out + (int64_t)(32 * mi + acc_row(v, lane)) * N + 32 * ni + (lane & 31));
  }
}

// Non-temporal 16-byte accesses for data that a kernel touches once.
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 stream_load4(const float* p) {
  const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void stream_store4(float* p, float4 v) {
  const f32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<f32x4*>(p));
}

// Four adjacent elements of a carried-state tensor, which is float32 or already rounded to
// bfloat16 (what the reference's combined forward hands from its state passing to its chunk scan,
// kernels/ema_combined.py:48-50: out_dtype = C.dtype).  STREAM: the non-temporal hint.
template <bool STREAM>
__device__ __forceinline__ float4 state_load4(const float* p) {
  return STREAM ? stream_load4(p) : *reinterpret_cast<const float4*>(p);
}
template <bool STREAM>
__device__ __forceinline__ float4 state_load4(const bf16_t* p) {
  const ema::bf16x4 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const ema::bf16x4*>(p))
                               : *reinterpret_cast<const ema::bf16x4*>(p);
  return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
}
__device__ __forceinline__ void state_store4(float* p, float4 v) { stream_store4(p, v); }
__device__ __forceinline__ void state_store4(bf16_t* p, float4 v) {
  const ema::bf16x4 w = {(bf16_t)v.x, (bf16_t)v.y, (bf16_t)v.z, (bf16_t)v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<ema::bf16x4*>(p));
}

// E adjacent elements of a state-sized tensor per thread: 4, or 8 where that makes the bfloat16
// accesses 16 bytes; a workgroup covers 256 * E elements of the state.
template <int E>
struct StateVec {
  float v[E];
};
template <int E>
__device__ __forceinline__ StateVec<E> state_load(const float* p) {
  StateVec<E> r;
#pragma unroll
  for (int i = 0; i < E; i += 4) {
    const float4 t = stream_load4(p + i);
    r.v[i] = t.x, r.v[i + 1] = t.y, r.v[i + 2] = t.z, r.v[i + 3] = t.w;
  }
  return r;
}
template <int E>
__device__ __forceinline__ StateVec<E> state_load(const bf16_t* p) {
  StateVec<E> r;
  if constexpr (E == 8) {
    const Vec16<bf16_t> t = load16_stream(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = t.get(i);
  } else {
    const float4 t = state_load4<true>(p);
    r.v[0] = t.x, r.v[1] = t.y, r.v[2] = t.z, r.v[3] = t.w;
  }
  return r;
}
template <int E>
__device__ __forceinline__ void state_store(float* p, const StateVec<E>& s) {
#pragma unroll
  for (int i = 0; i < E; i += 4) stream_store4(p + i, make_float4(s.v[i], s.v[i + 1], s.v[i + 2], s.v[i + 3]));
}
template <int E>
__device__ __forceinline__ void state_store(bf16_t* p, const StateVec<E>& s) {
  if constexpr (E == 8) {
    Vec16<bf16_t> t;
    t.set_all(s.v);
    store16_stream(p, t);
  } else {
    state_store4(p, make_float4(s.v[0], s.v[1], s.v[2], s.v[3]));
  }
}

// ------------------------------------------------------------------------------------
// state_passing.  out[b, c] = state entering chunk c, state <- exp(dA_chunk[c]) * state +
// states[b, c]; the value after the last chunk goes to final.  One thread per four adjacent
// state elements, the running state in registers, chunks fetched four ahead.
// states / out are (b, C, nh, dim) dense float32; dA_chunk is addressed by strides (it is the
// last column of dA_cumsum).  In a packed batch the state is dropped across a chunk whose last
// position has another id than the previous chunk's last position.
// ------------------------------------------------------------------------------------
template <typename TO, int E>
__global__ __launch_bounds__(256) void ssd_state_passing_kernel(
    const float* __restrict__ states, const float* __restrict__ dA_chunk, int64_t da_sb, int64_t da_sh,
    int64_t da_sc, const float* __restrict__ initial, TO* __restrict__ out, float* __restrict__ final_states,
    int nh, int C, int dim, int tiles, SeqIdx seq, int L, int Q) {
  const int tile = blockIdx.x % tiles;
  const int h = (blockIdx.x / tiles) % nh;
  const int64_t b = blockIdx.x / (tiles * nh);
  const int e = (tile * 256 + threadIdx.x) * E;
  if (e >= dim) return;
  const int64_t chunk_stride = (int64_t)nh * dim;
  const float* src = states + (b * C * nh + h) * (int64_t)dim + e;
  TO* dst = out + (b * C * nh + h) * (int64_t)dim + e;
  const float* da = dA_chunk + b * da_sb + h * da_sh;
  StateVec<E> s;
#pragma unroll
  for (int i = 0; i < E; ++i) s.v[i] = initial ? initial[(b * nh + h) * (int64_t)dim + e + i] : 0.f;
  constexpr int U = 4;
  for (int c0 = 0; c0 < C; c0 += U) {
    StateVec<E> nv[U];
    float a[U];
    // unconditional loads from chunk indices clamped into the tensor
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = min(c0 + u, C - 1);
      nv[u] = state_load<E>(src + c * chunk_stride);
      a[u] = __expf(da[(int64_t)c * da_sc]);
      if (!chunk_keeps_state(seq, b, c, Q, L)) a[u] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;
      if (c < C) {
        state_store<E>(dst + c * chunk_stride, s);
#pragma unroll
        for (int i = 0; i < E; ++i) s.v[i] = fmaf(a[u], s.v[i], nv[u].v[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < E; ++i) final_states[(b * nh + h) * (int64_t)dim + e + i] = s.v[i];
}

// ------------------------------------------------------------------------------------
// chunk_state and state_passing in one pass over x and B.  One workgroup (4 waves) per (b, h)
// walks the whole sequence in stages of 64 rows.  The local state of a chunk accumulates on MFMA
// exactly as in ssd_chunk_state_kernel (MODE 0); when a chunk ends the running state (float32, in
// the accumulator layout) becomes exp(dA_last) * state + local, as in ssd_state_passing_kernel, and
// when a chunk begins it is written out as the state entering that chunk.  The results equal those
// of the two kernels run one after the other bit for bit (same products in the same order, same
// fused multiply-add), while the chunk-local float32 states, twice the bytes of x, never touch
// memory.  The rows of D stages are in flight in registers at any time (a workgroup is alone on its
// compute unit and walks its rows in sequence, so the depth of this ring is what keeps its share
// of the memory system busy); LDS holds two stages, so a stage costs one barrier.  Q must be a
// multiple of 64 (a stage lies inside one chunk).  dt and dA_cs are (b, nh, C, Q), so position r of
// the sequence sits at offset r of the (b, h) row whatever the chunk.  No packed batches.
// ------------------------------------------------------------------------------------
template <typename T, int P, int NL>
struct WalkSmem {
  static constexpr int KT = 64, PX = Tile<T>::kpitch(P), PB = Tile<T>::kpitch(NL);
  static constexpr int kStageElems = KT * (PX + PB);
  static constexpr int kBytes = 2 * kStageElems * (int)sizeof(T);
};

// NSPLIT workgroups share one (b, h), each with N / NSPLIT columns of the state: with two of them
// per compute unit one multiplies while the other waits for its rows.  They read the same rows of
// x (adjacent workgroups, the same L2).
template <typename T, int P, int N, typename TO, int NSPLIT>
__global__ __launch_bounds__(256, NSPLIT) void ssd_state_walk_kernel(
    const T* __restrict__ x, Strides3 sx, const T* __restrict__ B, Strides3 sB, const float* __restrict__ dt,
    const float* __restrict__ dA_cs, const float* __restrict__ initial, TO* __restrict__ out,
    float* __restrict__ final_states, int nh, int heads_per_group, int L, int Q, int C) {
  constexpr int NL = N / NSPLIT;
  using S = WalkSmem<T, P, NL>;
  constexpr int KT = S::KT, PX = S::PX, PB = S::PB, KG = Tile<T>::KG;
  constexpr int MB = P / 32, NB = NL / 32, BPW = MB * NB / 4;
  static_assert(MB * NB % 4 == 0, "output blocks must split over 4 waves");
  // stages in flight: as many as the registers hold next to the two sets of accumulators
  constexpr int kPieceRegs = NSPLIT == 2
      ? (RowPieces<T, KT, P, S::PX>::CNT + RowPieces<T, KT, NL, S::PB>::CNT) * 6 + 2 * RowPieces<T, KT, NL, S::PB>::CNT
      : (RowPieces<T, KT, P, S::PX>::CNT + RowPieces<T, KT, NL, S::PB>::CNT) * 4 + 2 * RowPieces<T, KT, NL, S::PB>::CNT;
  constexpr int kRoom = 256 - 2 * BPW * 16 - (NSPLIT == 2 ? 140 : 40 + 8 * BPW + (sizeof(T) == 4 ? 16 : 0));
#ifdef SSD_WALK_D
  constexpr int D = SSD_WALK_D;
#else
  constexpr int D = kRoom >= 4 * kPieceRegs ? 4 : (kRoom >= 3 * kPieceRegs ? 3 : (kRoom >= 2 * kPieceRegs ? 2 : 1));
#endif
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* lds = reinterpret_cast<T*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int part = bid % NSPLIT;
  const int h = (bid / NSPLIT) % nh;
  const int64_t b = bid / (NSPLIT * nh);
  const int n0 = part * NL;  // first state column of this workgroup
  const float* dAb = dA_cs + (b * nh + h) * (int64_t)C * Q;
  const float* dtb = dt + (b * nh + h) * (int64_t)C * Q;
  const T* xg = x + b * sx.sb + h * sx.sh;
  const T* Bg = B + b * sB.sb + (h / heads_per_group) * sB.sh + n0;
  const int G = (L + KT - 1) / KT;

  // element (p, n) of the state <-> accumulator i, component v of this lane
  auto elem = [&](int i, int v) {
    const int j = wave + 4 * i, mi = j % MB, ni = j / MB;
    return (32 * mi + acc_row(v, lane)) * N + n0 + 32 * ni + (lane & 31);
  };
  // Every request is unconditional (a load inside a branch would have to complete before the next
  // is issued): stages past the end are requested again as the last one and never used.
  RowPieces<T, KT, P, S::PX> px[D];
  RowPieces<T, KT, NL, S::PB> pb[D];
  auto request = [&](RowPieces<T, KT, P, S::PX>& rx, RowPieces<T, KT, NL, S::PB>& rb, int g) {
    const int row0 = min(g, G - 1) * KT;
#ifndef SSD_WALK_XNT
#define SSD_WALK_XNT true
#endif
    rx.template load<SSD_WALK_XNT>(xg, sx.sl, row0, L, tid);
    rb.template load<false, true>(Bg, sB.sl, row0, L, tid, dAb, dtb);
  };
#pragma unroll
  for (int u = 0; u < D; ++u) request(px[u], pb[u], u);

  floatx16 acc[BPW], st[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    zero_acc(acc[i]);
    zero_acc(st[i]);
  }
  if (initial) {
    const float* ini = initial + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) st[i][v] = ini[elem(i, v)];
  }
  // the decay sum at the end of the chunk a stage belongs to, fetched one chunk ahead
  float dal_next = dAb[Q - 1], dal = 0.f;

  // one stage: rx / rb hold its rows and receive those of stage g + D
  auto stage = [&](RowPieces<T, KT, P, S::PX>& rx, RowPieces<T, KT, NL, S::PB>& rb, int g) {
    const int row0 = g * KT;
    const int c = row0 / Q, k0 = row0 - c * Q;
    if (k0 == 0) {
      dal = dal_next;
      dal_next = dAb[(int64_t)min(c + 1, C - 1) * Q + Q - 1];
      TO* o = out + ((b * C + c) * nh + h) * (int64_t)(P * N);
#pragma unroll
      for (int i = 0; i < BPW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) __builtin_nontemporal_store((TO)st[i][v], o + elem(i, v));
    }
    T* xb = lds + (g & 1) * S::kStageElems;
    T* bb = xb + KT * PX;
    const float dA_last = dal;
    rx.store(xb, row0, L, tid, NoScale());
    rb.store(bb, row0, L, tid, [&](int, float dA_k, float dt_k) { return __expf(fminf(dA_last - dA_k, 0.f)) * dt_k; });
    __syncthreads();
    request(rx, rb, g + D);
#pragma unroll
    for (int kk = 0; kk < KT; kk += KG) {
#pragma unroll
      for (int i = 0; i < BPW; ++i) {
        const int j = wave + 4 * i, mi = j % MB, ni = j / MB;
        mma_group(frag_cols(xb, PX, kk, 32 * mi, lane), frag_cols(bb, PB, kk, 32 * ni, lane), acc[i]);
      }
    }
    if (k0 + KT >= Q || g == G - 1) {  // the chunk ends with this stage
      const float a = __expf(dA_last);
#pragma unroll
      for (int i = 0; i < BPW; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) st[i][v] = fmaf(a, st[i][v], acc[i][v]);
        zero_acc(acc[i]);
      }
    }
  };
  // Whole rounds of D stages run without a test between the stages: every path through a round
  // issues the same loads, so the waits for a stage's rows leave the rounds behind it in flight.
  int g0 = 0;
  for (; g0 + D <= G; g0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) stage(px[u], pb[u], g0 + u);
  }
#pragma unroll
  for (int u = 0; u < D - 1; ++u)
    if (g0 + u < G) stage(px[u], pb[u], g0 + u);
  float* f = final_states + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
  for (int i = 0; i < BPW; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) f[elem(i, v)] = st[i][v];
}

// ------------------------------------------------------------------------------------
// The same walk for bfloat16, hdim 64, dstate 128, with the rows copied from global memory straight
// into LDS.  A workgroup is alone on its compute unit and walks its rows in sequence, so what keeps
// its share of the memory system busy is the number of stages in flight; copies into LDS occupy no
// registers, which also leaves room for eight waves (one 32 x 32 block of the state each) where the
// register-staged kernel has four.  R stages live in LDS: while stage g is multiplied the copies of
// stages g + 1 .. g + R - 1 are under way; one barrier per stage.  Per stage: 64 rows of x (128-byte
// rows) and of B (256-byte rows), both read with the transposing read and therefore stored with
// their 16-byte pieces permuted (see the dB / dC kernel below), and two small pieces with the stage's dA
// and dt and the chunk's last dA.  B arrives unweighted, so the weight exp(min(dA_last - dA_k, 0)) dt_k
// is applied to the operand fragment (float32 product, rounded to bfloat16: the same arithmetic as where
// the register-staged kernels weight the rows on their way into LDS); each wave computes the stage's 64
// weights once, a lane each, and passes them through 256 bytes of LDS of its own.  Results equal those
// of the register-staged kernel (and of the two launchers) bit for bit.
//
// The waits are placed by hand.  Copies and stores of a wave complete in the order of their requests,
// and the counter that s_waitcnt vmcnt(n) tests counts both; a stage's copies have landed once no more
// than the requests made after them are outstanding: three copies for each later stage in flight (a
// wave requests three or four per stage) and the sixteen stores of the state entering a chunk, if a
// chunk began since.  No ordinary load may sit in the loop: its wait would wait for every copy before
// it as well.
// ------------------------------------------------------------------------------------
struct WalkDmaSmem {
  static constexpr int R = 4;  // stages in LDS (five and six measured slower)
  static constexpr int kX = 64 * 64 * (int)sizeof(bf16_t), kB = 64 * 128 * (int)sizeof(bf16_t), kVec = 2048;
  static constexpr int kStage = kX + kB + kVec;
  static constexpr int kBytes = R * kStage + 8 * 64 * (int)sizeof(float);  // + the weights, a copy per wave
};

template <typename TO>
__global__ __launch_bounds__(512) void ssd_state_walk_dma_kernel(
    const bf16_t* __restrict__ x, Strides3 sx, const bf16_t* __restrict__ B, Strides3 sB, const float* __restrict__ dt,
    const float* __restrict__ dA_cs, const float* __restrict__ initial, TO* __restrict__ out,
    float* __restrict__ final_states, int nh, int heads_per_group, int L, int Q, int C) {
  using S = WalkDmaSmem;
  using T = bf16_t;
  constexpr int P = 64, N = 128, KT = 64, KG = 16, MB = P / 32, R = S::R;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5;
  float* wl = reinterpret_cast<float*>(smem + R * S::kStage) + wave * 64;  // this wave's copy of the weights
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int h = bid % nh;
  const int64_t b = bid / nh;
  const float* dAb = dA_cs + (b * nh + h) * (int64_t)C * Q;
  const float* dtb = dt + (b * nh + h) * (int64_t)C * Q;
  const T* xg = x + b * sx.sb + h * sx.sh;
  const T* Bg = B + b * sB.sb + (h / heads_per_group) * sB.sh;
  const int G = (L + KT - 1) / KT;
  const int mi = wave % MB, ni = wave / MB;  // this wave's block of the state: rows 32 mi .., columns 32 ni ..
  auto elem = [&](int v) { return (32 * mi + acc_row(v, lane)) * N + 32 * ni + (lane & 31); };

  // The copies of stage g into LDS set u: wave w brings rows 8 w .. 8 w + 7 of x (one instruction),
  // rows 8 w .. of B (two), and waves 0 / 1 the pieces of dA / dt.  What depends on the lane is
  // computed here; a request moves scalar bases (and clamps the rows of the last, ragged stage).
  // Copies a wave requests per stage: kXCopies of x, kBCopies of B (and one more on waves 0 / 1).  The
  // hand-placed waits below count on exactly these numbers.
  constexpr int kXCopies = 1, kBCopies = 2, kMinCopies = kXCopies + kBCopies;
  constexpr int kStateStores = 16;  // stores of the state entering a chunk, per lane
  static_assert(8 * 8 * kXCopies == KT && 8 * 4 * kBCopies == KT, "eight waves bring the 64 rows of a stage");
  static_assert(sizeof(floatx16) == kStateStores * sizeof(float), "one store per accumulator register");
  const int xr = 8 * wave + (lane >> 3);                                  // row of x inside the stage
  const unsigned x_piece = 16u * ((lane & 7) ^ (4 * ((xr >> 1) & 1)));    // byte offset inside the row
  int br[kBCopies];
  unsigned b_piece[kBCopies];
#pragma unroll
  for (int j = 0; j < kBCopies; ++j) {
    br[j] = 4 * (2 * wave + j) + (lane >> 4);
    b_piece[j] = 16u * ((lane & 15) ^ (4 * (br[j] & 3)));
  }
  auto request = [&](int g, int u) {
    const int row0 = min(g, G - 1) * KT;
    const int last = L - 1 - row0;  // rows past the sequence repeat its last row (their weight is 0)
    unsigned char* base = smem + u * S::kStage;
    copy16_to_lds(xg + (int64_t)row0 * sx.sl, (unsigned)(min(xr, last) * sx.sl) * 2u + x_piece, base + wave * 1024);
    const T* bg = Bg + (int64_t)row0 * sB.sl;
#pragma unroll
    for (int j = 0; j < kBCopies; ++j)
      copy16_to_lds(bg, (unsigned)(min(br[j], last) * sB.sl) * 2u + b_piece[j], base + S::kX + (2 * wave + j) * 1024);
    if (wave < 2) {
      // lanes 0 .. 15: the stage's 64 values; the others: the chunk's last four values of dA (dt: anything valid)
      const int tail = (row0 / Q + 1) * Q - 4 - row0;
      const unsigned off = 4u * (unsigned)(lane < 16 ? 4 * lane : (wave == 0 ? tail : 0));
      copy16_to_lds((wave == 0 ? dAb : dtb) + row0, off, base + S::kX + S::kB + wave * 1024);
    }
  };
#pragma unroll
  for (int u = 0; u < R - 1; ++u) request(u, u);

  floatx16 acc, st;
  zero_acc(acc);
  zero_acc(st);
  if (initial) {
    const float* ini = initial + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
    for (int v = 0; v < 16; ++v) st[v] = ini[elem(v)];
  }
  // (waited for here, so that no wait for ordinary loads falls into the loop)
#pragma unroll
  for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(st[v]));

  // where this lane reads its operand fragments inside a stage's tiles (elements)
  int x_off, b_off;
  {
    const int i16 = lane & 15;
    const int row = 8 * half + (i16 >> 2);
    const int cx = 32 * mi + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    const int cb = 32 * ni + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    x_off = row * P + 8 * ((cx >> 3) ^ (4 * ((row >> 1) & 1))) + (cx & 7);
    b_off = row * N + 8 * ((cb >> 3) ^ (4 * (row & 3))) + (cb & 7);
  }
  typedef __attribute__((address_space(3))) ema::bf16x4 lds_bf16x4;
  auto tr_read = [&](const T* p, int pitch) {
    const ema::bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
    const ema::bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * pitch));  // row + 4: the same key
    Vec16<T> r;
    r.raw = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return r;
  };

  int since = R;  // stages since the last chunk began (at least R: no stores in the queue)
  for (int g = 0; g < G; ++g) {
    const int u = g % R;
    const int row0 = g * KT;
    const int c = row0 / Q, k0 = row0 - c * Q;
    // The copies of this stage have landed once only later requests are outstanding: those of the R - 2
    // stages after it (three per wave and stage, four for two of the waves) and, if a chunk began
    // 1 .. R - 2 stages ago, the sixteen stores of its entering state (with chunks of one or two stages
    // there may be two such chunks: the lower count waits a little longer).
    static_assert(kMinCopies * (R - 2) + kStateStores < 64, "the counter holds 6 bits");
    if (since <= R - 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kMinCopies * (R - 2) + kStateStores) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kMinCopies * (R - 2)) : "memory");
    __syncthreads();  // every wave's part of the stage is there; every wave is done with stage g - 1
    if (k0 == 0) {  // the state entering the chunk
      TO* o = out + ((b * C + c) * nh + h) * (int64_t)(P * N);
#pragma unroll
      for (int v = 0; v < kStateStores; ++v) __builtin_nontemporal_store((TO)st[v], o + elem(v));
      since = 0;
    }
    ++since;
    request(g + R - 1, (g + R - 1) % R);
    const unsigned char* base = smem + u * S::kStage;
    const T* xb = reinterpret_cast<const T*>(base);
    const T* bb = reinterpret_cast<const T*>(base + S::kX);
    const float* vec = reinterpret_cast<const float*>(base + S::kX + S::kB);  // dA rows, dA tail | dt rows
    const float dA_last = vec[67];
    wl[lane] = __expf(fminf(dA_last - vec[lane], 0.f)) * vec[256 + lane];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // the wave's own LDS writes are visible to its own reads
#pragma unroll
    for (int ks = 0; ks < KT / KG; ++ks) {
      const Vec16<T> xf = tr_read(xb + x_off + KG * ks * P, P);
      Vec16<T> bf = tr_read(bb + b_off + KG * ks * N, N);
      float t[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) t[e] = bf.get(e) * wl[KG * ks + 8 * half + e];
      bf.set_all(t);
      mma_group(xf, bf, acc);
    }
    if (k0 + KT >= Q || g == G - 1) {  // the chunk ends with this stage
      const float a = __expf(dA_last);
#pragma unroll
      for (int v = 0; v < 16; ++v) st[v] = fmaf(a, st[v], acc[v]);
      zero_acc(acc);
    }
  }
  float* f = final_states + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
  for (int v = 0; v < 16; ++v) f[elem(v)] = st[v];
}

// ------------------------------------------------------------------------------------
// The mirror image of that walk for the backward: the gradient of the chunk scan with respect to
// the carried states (MODE 1 of ssd_chunk_state_kernel) and the reverse recurrence over the chunks
// (ssd_state_passing_bwd_kernel) in one kernel, for bfloat16, hdim 64, dstate 128, bfloat16 carried
// states and chunks of at least two stages.  A workgroup per (b, h) walks the chunks from the last
// to the first (the 64-row stages of a chunk in ascending order, as the stage kernel sums them) with
//   D_c   = sum_k round(dout[k] * exp(dA_k)) (x) C[k]          over the rows of chunk c (accumulators)
//   dstates[c] = G,   part[(b,h,c), wave] = <states[c], G>     at the chunk's first stage
//   G     = exp(dA_chunk[c]) * G + D_c                          at its last
// where G starts from dfinal (or zero) and ends as dinit.  D_c never leaves the accumulators: the
// float32 (or rounded) copy that the two launchers write and read back is gone, and the results
// are those of the two launchers with a float32 D_c (dstates bit for bit; the per-chunk dots are
// summed in another order).  The finish kernel of the state passing turns the partial dots into ddA.
//
// Rows arrive as in the forward walk: R stages of dout (128-byte rows), C (256-byte rows) and dA in
// LDS by direct copies, the waits placed by hand.  states[c] (16 KB) comes the same way with the
// request of the chunk's first stage, ahead of that stage's rows, into one of three buffers in turn:
// the buffer of chunk c was read last at the first stage of chunk c + 3, at least six steps before
// this request (chunks have two stages or more), and the request is made behind a barrier that every
// wave passes after that step.  Counting: a wave requests kMinCopies copies per stage or more (two
// for the state tile, one for dA), so once no more than kMinCopies * (R - 2) requests are
// outstanding everything up to this stage's rows has landed; the stores of a chunk's first stage
// (sixteen of dstates and one partial dot) share the counter and are allowed for while they can
// still be in the queue.
// ------------------------------------------------------------------------------------
struct WalkBwdDmaSmem {
  static constexpr int R = WalkDmaSmem::R;
  static constexpr int kX = WalkDmaSmem::kX, kB = WalkDmaSmem::kB, kVec = 1024;
  static constexpr int kStage = kX + kB + kVec;
  static constexpr int kWeights = 8 * 64 * (int)sizeof(float);
  static constexpr int kTile = 64 * 128 * (int)sizeof(bf16_t), kTiles = 3;
  static constexpr int kBytes = R * kStage + kWeights + kTiles * kTile;
};

template <typename TG>
__global__ __launch_bounds__(512) void ssd_state_walk_bwd_dma_kernel(
    const bf16_t* __restrict__ dout, Strides3 sx, const bf16_t* __restrict__ Cm, Strides3 sC,
    const float* __restrict__ dA_cs, const bf16_t* __restrict__ states, const float* __restrict__ dfinal,
    TG* __restrict__ dstates, float* __restrict__ part, float* __restrict__ dinit, int nh, int heads_per_group, int L,
    int Q, int C) {
  using S = WalkBwdDmaSmem;
  using T = bf16_t;
  constexpr int P = 64, N = 128, KT = 64, KG = 16, MB = P / 32, R = S::R;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), half = lane >> 5;
  float* wl = reinterpret_cast<float*>(smem + R * S::kStage) + wave * 64;  // this wave's copy of the weights
  unsigned char* tiles = smem + R * S::kStage + S::kWeights;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int h = bid % nh;
  const int64_t b = bid / nh;
  const float* dAb = dA_cs + (b * nh + h) * (int64_t)C * Q;
  const T* xg = dout + b * sx.sb + h * sx.sh;
  const T* Cg = Cm + b * sC.sb + (h / heads_per_group) * sC.sh;
  const int SPC = Q / KT;                              // stages of a whole chunk
  const int S_last = (L - (C - 1) * Q + KT - 1) / KT;  // stages of the last chunk, which comes first
  const int G = S_last + (C - 1) * SPC;
  const int mi = wave % MB, ni = wave / MB;  // this wave's block of the state: rows 32 mi .., columns 32 ni ..
  auto elem = [&](int v) { return (32 * mi + acc_row(v, lane)) * N + 32 * ni + (lane & 31); };
  // step i of the walk works on stage s of chunk c
  auto stage_of = [&](int i, int& c, int& s) {
    if (i < S_last) {
      c = C - 1, s = i;
    } else {
      const int j = i - S_last;
      c = C - 2 - j / SPC, s = j % SPC;
    }
  };

  constexpr int kXCopies = 1, kCCopies = 2, kMinCopies = kXCopies + kCCopies, kTileCopies = 2;
  constexpr int kChunkStores = 16 + 1;  // dstates, and the wave's partial dot
  static_assert(8 * 8 * kXCopies == KT && 8 * 4 * kCCopies == KT, "eight waves bring the 64 rows of a stage");
  static_assert(8 * kTileCopies * 1024 == S::kTile, "eight waves bring the state tile");
  static_assert(sizeof(floatx16) == (kChunkStores - 1) * sizeof(float), "one store per accumulator register");
  const int xr = 8 * wave + (lane >> 3);                                  // row of dout inside the stage
  const unsigned x_piece = 16u * ((lane & 7) ^ (4 * ((xr >> 1) & 1)));    // byte offset inside the row
  int cr[kCCopies];
  unsigned c_piece[kCCopies];
#pragma unroll
  for (int j = 0; j < kCCopies; ++j) {
    cr[j] = 4 * (2 * wave + j) + (lane >> 4);
    c_piece[j] = 16u * ((lane & 15) ^ (4 * (cr[j] & 3)));
  }
  auto request = [&](int i, int u) {
    int c, s;
    stage_of(min(i, G - 1), c, s);
    const int row0 = c * Q + s * KT;
    const int last = L - 1 - row0;  // rows past the sequence repeat its last row (their weight is 0)
    unsigned char* base = smem + u * S::kStage;
    if (s == 0 && i < G) {  // the state entering the chunk, ahead of the rows
      const T* sg = states + ((b * C + c) * nh + h) * (int64_t)(P * N) + wave * (kTileCopies * 512);
      unsigned char* dst = tiles + (c % S::kTiles) * S::kTile + wave * (kTileCopies * 1024);
#pragma unroll
      for (int j = 0; j < kTileCopies; ++j) copy16_to_lds(sg + j * 512, 16u * (unsigned)lane, dst + j * 1024);
    }
    copy16_to_lds(xg + (int64_t)row0 * sx.sl, (unsigned)(min(xr, last) * sx.sl) * 2u + x_piece, base + wave * 1024);
    const T* cg = Cg + (int64_t)row0 * sC.sl;
#pragma unroll
    for (int j = 0; j < kCCopies; ++j)
      copy16_to_lds(cg, (unsigned)(min(cr[j], last) * sC.sl) * 2u + c_piece[j], base + S::kX + (2 * wave + j) * 1024);
    if (wave == 0) {
      // lanes 0 .. 15: the stage's 64 values of dA; the others: the chunk's last four
      const int tail = (c + 1) * Q - 4 - row0;
      copy16_to_lds(dAb + row0, 4u * (unsigned)(lane < 16 ? 4 * lane : tail), base + S::kX + S::kB);
    }
  };
#pragma unroll
  for (int u = 0; u < R - 1; ++u) request(u, u);

  floatx16 acc, gr;
  zero_acc(acc);
  zero_acc(gr);
  if (dfinal) {
    const float* fin = dfinal + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
    for (int v = 0; v < 16; ++v) gr[v] = fin[elem(v)];
  }
  // (waited for here, so that no wait for ordinary loads falls into the loop)
#pragma unroll
  for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(gr[v]));

  // where this lane reads its operand fragments inside a stage's tiles (elements)
  int x_off, c_off;
  {
    const int i16 = lane & 15;
    const int row = 8 * half + (i16 >> 2);
    const int cx = 32 * mi + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    const int cc = 32 * ni + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    x_off = row * P + 8 * ((cx >> 3) ^ (4 * ((row >> 1) & 1))) + (cx & 7);
    c_off = row * N + 8 * ((cc >> 3) ^ (4 * (row & 3))) + (cc & 7);
  }
  typedef __attribute__((address_space(3))) ema::bf16x4 lds_bf16x4;
  auto tr_read = [&](const T* p, int pitch) {
    const ema::bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
    const ema::bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * pitch));  // row + 4: the same key
    Vec16<T> r;
    r.raw = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return r;
  };

  int since = R;  // steps since the last chunk began (at least R: no stores in the queue)
  for (int i = 0; i < G; ++i) {
    const int u = i % R;
    int c, s;
    stage_of(i, c, s);
    const int row0 = c * Q + s * KT;
    static_assert(kMinCopies * (R - 2) + kChunkStores < 64, "the counter holds 6 bits");
    if (since <= R - 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kMinCopies * (R - 2) + kChunkStores) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kMinCopies * (R - 2)) : "memory");
    __syncthreads();  // every wave's part of the stage is there; every wave is done with step i - 1
    if (s == 0) {  // dstates[c] and the wave's share of <states[c], G>
      TG* o = dstates + ((b * C + c) * nh + h) * (int64_t)(P * N);
      const T* tile = reinterpret_cast<const T*>(tiles + (c % S::kTiles) * S::kTile);
      float dot = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        __builtin_nontemporal_store((TG)gr[v], o + elem(v));
        dot = fmaf((float)tile[elem(v)], gr[v], dot);
      }
      dot = ema::wave_sum(dot);
      if (lane == 0) part[((b * nh + h) * (int64_t)C + c) * 8 + wave] = dot;
      since = 0;
    }
    ++since;
    request(i + R - 1, (i + R - 1) % R);
    const unsigned char* base = smem + u * S::kStage;
    const T* xb = reinterpret_cast<const T*>(base);
    const T* cb = reinterpret_cast<const T*>(base + S::kX);
    const float* vec = reinterpret_cast<const float*>(base + S::kX + S::kB);  // dA of the rows, dA tail
    const float dA_last = vec[67];
    wl[lane] = row0 + lane < L ? __expf(vec[lane]) : 0.f;
    __builtin_amdgcn_s_waitcnt(0xc07f);  // the wave's own LDS writes are visible to its own reads
#pragma unroll
    for (int ks = 0; ks < KT / KG; ++ks) {
      Vec16<T> xf = tr_read(xb + x_off + KG * ks * P, P);
      const Vec16<T> cf = tr_read(cb + c_off + KG * ks * N, N);
      float t[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) t[e] = xf.get(e) * wl[KG * ks + 8 * half + e];
      xf.set_all(t);
      mma_group(xf, cf, acc);
    }
    if (s == (c == C - 1 ? S_last : SPC) - 1) {  // the chunk ends with this stage
      const float a = __expf(dA_last);
#pragma unroll
      for (int v = 0; v < 16; ++v) gr[v] = fmaf(a, gr[v], acc[v]);
      zero_acc(acc);
    }
  }
  if (dinit) {
    float* f = dinit + (b * nh + h) * (int64_t)(P * N);
#pragma unroll
    for (int v = 0; v < 16; ++v) f[elem(v)] = gr[v];
  }
}

// Sum over the 32 lanes of each half of a wave (lanes 0..31 and 32..63 apart), left in lanes 31
// and 63: the DPP prefix steps of wave_inclusive_scan without the last one.
__device__ __forceinline__ float half_wave_sum(float v) {
  v += ema::dpp_or_zero<0x111, 0xf>(v);
  v += ema::dpp_or_zero<0x112, 0xf>(v);
  v += ema::dpp_or_zero<0x114, 0xf>(v);
  v += ema::dpp_or_zero<0x118, 0xf>(v);
  v += ema::dpp_or_zero<0x142, 0xa>(v);
  return v;
}

// ------------------------------------------------------------------------------------
// state_passing backward.  With G the gradient of the state entering the next chunk (G starts
// from dfinal or 0): dstates[c] = G, part[(b,h,c), wave] = <states[c], G> over the wave's
// elements, G <- exp(dA_chunk[c]) * G + dout[c]; after chunk 0, G goes to dinit if asked.
// The finish kernel sums the wave partials: ddA[b,h,c] = exp(dA_chunk[c]) * sum, and 0 for
// c = 0 when there is no initial state.
// ------------------------------------------------------------------------------------
template <typename TS, typename TD, typename TG, int E>
__global__ __launch_bounds__(256) void ssd_state_passing_bwd_kernel(
    const TS* __restrict__ states, const float* __restrict__ dA_chunk, int64_t da_sb, int64_t da_sh,
    int64_t da_sc, const TD* __restrict__ dout, const float* __restrict__ dfinal,
    TG* __restrict__ dstates, float* __restrict__ part, float* __restrict__ dinit, int nh, int C, int dim,
    int tiles, SeqIdx seq, int L, int Q) {
  const int tile = blockIdx.x % tiles;
  const int h = (blockIdx.x / tiles) % nh;
  const int64_t b = blockIdx.x / (tiles * nh);
  const int e = (tile * 256 + threadIdx.x) * E;
  const bool ok = e < dim;
  const int lane = threadIdx.x & 63;
  const int wave_id = tile * 4 + (threadIdx.x >> 6), nw = tiles * 4;
  const int64_t chunk_stride = (int64_t)nh * dim;
  const int64_t base = (b * C * nh + h) * (int64_t)dim + (ok ? e : 0);
  const float* da = dA_chunk + b * da_sb + h * da_sh;
  StateVec<E> G;
#pragma unroll
  for (int i = 0; i < E; ++i) G.v[i] = (dfinal && ok) ? dfinal[(b * nh + h) * (int64_t)dim + e + i] : 0.f;
  constexpr int U = 4;
  for (int c1 = C - 1; c1 >= 0; c1 -= U) {
    StateVec<E> sv[U], dv[U];
    float a[U];
    // unconditional loads from chunk indices clamped into the tensor; what lies outside is zeroed
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = max(c1 - u, 0);
      sv[u] = state_load<E>(states + base + c * chunk_stride);
      dv[u] = state_load<E>(dout + base + c * chunk_stride);
      a[u] = __expf(da[(int64_t)c * da_sc]);
      if (!chunk_keeps_state(seq, b, c, Q, L)) a[u] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c1 - u;
      if (c >= 0) {  // uniform across the workgroup
        if (ok) state_store<E>(dstates + base + c * chunk_stride, G);
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < E; ++i) dot = fmaf(sv[u].v[i], G.v[i], dot);
        dot = ema::wave_sum(ok ? dot : 0.f);
        if (lane == 0) part[((b * nh + h) * C + c) * (int64_t)nw + wave_id] = dot;
#pragma unroll
        for (int i = 0; i < E; ++i) G.v[i] = fmaf(a[u], G.v[i], dv[u].v[i]);
      }
    }
  }
  if (dinit && ok) {
#pragma unroll
    for (int i = 0; i < E; ++i) dinit[(b * nh + h) * (int64_t)dim + e + i] = G.v[i];
  }
}

__global__ __launch_bounds__(256) void ssd_state_passing_bwd_finish_kernel(
    const float* __restrict__ part, const float* __restrict__ dA_chunk, int64_t da_sb, int64_t da_sh,
    int64_t da_sc, float* __restrict__ ddA, int nh, int C, int nw, int has_init, int64_t total, SeqIdx seq,
    int L, int Q) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (b * nh + h) * C + c
  if (i >= total) return;
  const int c = (int)(i % C);
  const int64_t bh = i / C;
  const int h = (int)(bh % nh);
  const int64_t b = bh / nh;
  float s = 0.f;
  for (int w = 0; w < nw; ++w) s += part[i * nw + w];
  const bool dropped = (c == 0 && !has_init) || !chunk_keeps_state(seq, b, c, Q, L);
  ddA[i] = dropped ? 0.f : __expf(dA_chunk[b * da_sb + h * da_sh + (int64_t)c * da_sc]) * s;
}

// In-place inclusive cumsum along the last axis of a dense (rows, Q) float32 array; one wave
// per row, lane l owns ceil(Q/64) consecutive positions.
__global__ __launch_bounds__(256) void ssd_row_cumsum_kernel(float* __restrict__ v, int Q, int64_t rows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int per = (Q + 63) >> 6;
  float* p = v + row * Q;
  float local = 0.f;
  for (int i = 0; i < per; ++i) {
    const int q = lane * per + i;
    if (q < Q) local += p[q];
  }
  float run = wave_inclusive_scan(local) - local;
  for (int i = 0; i < per; ++i) {
    const int q = lane * per + i;
    if (q < Q) {
      run += p[q];
      p[q] = run;
    }
  }
}

// ------------------------------------------------------------------------------------
// Gradients that are summed over the heads of a group: dB (MODE 0) and the carried-state part
// of dC (MODE 1).  One workgroup per (b, c, g, tile of 64 rows m), looping over the group's heads:
//   per head   d_h[m][n] = (sum_p a[m][p] * round_T(s[p][n])) * w_m
//     MODE 0:  a = x,    s = dstates, w_m = exp(min(dA_last - dA_m, 0)) * dt_m
//     MODE 1:  a = dout, s = prev,    w_m = exp(dA_m)
//   out[m][n] = sum_h d_h[m][n]                       (float32, (b, L, g, N))
//   with bc (B for MODE 0, C for MODE 1): r_h[m] = sum_n d_h[m][n] * bc[m][n], written to
//   ddA[b,h,c, m + 1] (MODE 0, slot 0 = 0; the caller then takes the cumsum) or ddA[b,h,c,m] (MODE 1).
// In a packed batch w_m is 0 unless the id of m equals the id of the chunk's last position
// (MODE 0) or of the previous chunk's last position (MODE 1).
// a is read row-major straight from global memory; s is staged in LDS (rounded to T) and
// contracted along its rows.  The products are formed transposed, d_h^T = s^T a^T, so that in
// the accumulator a lane owns one row m and sixteen columns n: the row weight is one value per
// lane and the sum over n for r_h is in-register adds, one exchange between the halves of the
// wave and one between two waves through LDS (summing the untransposed accumulator across
// lanes took as long as everything else in the kernel).
// ------------------------------------------------------------------------------------
template <typename T, int P, int N>
struct GroupSmem {
  static constexpr int PS = Tile<T>::kpitch(N);  // the state tile is contracted along its rows
  static constexpr int kBytes = P * PS * (int)sizeof(T) + (4 * 64 + 64) * (int)sizeof(float);
};

template <typename T, int P, int N, int MODE, typename TS>
__global__ __launch_bounds__(256) void ssd_group_grad_kernel(
    const T* __restrict__ a, Strides3 sa, const TS* __restrict__ s, const float* __restrict__ dt,
    const float* __restrict__ dA_cs, const T* __restrict__ bc, Strides3 sbc, float* __restrict__ out,
    float* __restrict__ ddA, int nh, int heads_per_group, int ngroups, int L, int Q, int C, int mtiles,
    SeqIdx seq) {
  using S = GroupSmem<T, P, N>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, NB = N / 32, BPW = 2 * NB / 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* St = reinterpret_cast<T*>(smem);
  float* rs = reinterpret_cast<float*>(smem + P * S::PS * sizeof(T));  // [4 waves][64 rows]
  float* wrow = rs + 4 * 64;                                           // this head's row weights

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int mt = bid % mtiles;
  const int g = (bid / mtiles) % ngroups;
  const int c = (bid / (mtiles * ngroups)) % C;
  const int64_t b = bid / ((int64_t)mtiles * ngroups * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = 64 * mt;

  // packed batch: rows of another sequence than the reference position get no weight
  bool row_live = true;
  {
    const ChunkSeq sq = chunk_seq(seq, b, c, Q);
    if (sq.on() && tid < 64) {
      const int ref = MODE == 0 ? sq.at(limit - 1) : sq.entering(c);
      row_live = sq.at(min(m0 + tid, limit - 1)) == ref;
    }
  }
  // block i of this wave: rows 32*mi.., columns 32*ni..
  int mi[BPW], ni[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int j = wave + 4 * i;
    mi[i] = j & 1;
    ni[i] = j >> 1;
  }
  // bc in the (transposed) accumulator layout: this lane's row m, columns n of each block
  float bcv[BPW][16];
  const bool want_ddA = bc != nullptr;
  if (want_ddA) {
    const T* bcg = bc + b * sbc.sb + (int64_t)c * Q * sbc.sl + g * sbc.sh;
    const int m = m0 + 32 * mi[0] + l32;
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float t = (float)bcg[(int64_t)min(m, limit - 1) * sbc.sl + 32 * ni[i] + acc_row(v, lane)];
        bcv[i][v] = m < limit ? t : 0.f;
      }
  }
  floatx16 total[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) zero_acc(total[i]);

  for (int hh = 0; hh < heads_per_group; ++hh) {
    const int h = g * heads_per_group + hh;
    const int64_t chunk = (b * nh + h) * C + c;
    const float* dAp = dA_cs + chunk * Q;
    const float* dtp = dt + chunk * Q;
    const TS* sg = s + (((b * C + c) * nh + h) * (int64_t)P) * N;
    const T* ag = a + b * sa.sb + (int64_t)c * Q * sa.sl + h * sa.sh;
    // every global load of this head goes out here, before the first wait: the state tile, the
    // wave's rows of a (its blocks share them), the row weights
    constexpr int VPR = N / 4, NLD = P * VPR / 256, KS = P / KG;
    float4 sv[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + 256 * i;
      sv[i] = state_load4<false>(sg + (int64_t)(idx / VPR) * N + (idx % VPR) * 4);
    }
    const int m_lane = m0 + 32 * mi[0] + l32;
    Vec16<T> av[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      av[ks] = load16(ag + (int64_t)min(m_lane, limit - 1) * sa.sl + KG * ks + EPL * half);
    float wv = 0.f;
    if (tid < 64) {  // one weight per row, computed once instead of by every lane that holds the row
      const int mc = min(m0 + tid, Q - 1);
      wv = MODE == 0 ? __expf(fminf(dAp[Q - 1] - dAp[mc], 0.f)) * dtp[mc] : __expf(dAp[mc]);
      wrow[tid] = (m0 + tid < Q && row_live) ? wv : 0.f;
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int idx = tid + 256 * i;
      T* d = St + (idx / VPR) * S::PS + (idx % VPR) * 4;
      d[0] = (T)sv[i].x, d[1] = (T)sv[i].y, d[2] = (T)sv[i].z, d[3] = (T)sv[i].w;
    }
    __syncthreads();
    floatx16 acc[BPW];
#pragma unroll
    for (int i = 0; i < BPW; ++i) zero_acc(acc[i]);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (m_lane >= limit) av[ks].zero();
#pragma unroll
      for (int i = 0; i < BPW; ++i)
        mma_group(frag_cols(St, S::PS, KG * ks, 32 * ni[i], lane), av[ks], acc[i]);  // [n][m]
    }
    {
      const float w = wrow[32 * mi[0] + l32];  // the wave's blocks share their rows m
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < BPW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          total[i][v] = fmaf(acc[i][v], w, total[i][v]);
          if (want_ddA) part = fmaf(acc[i][v], bcv[i][v], part);
        }
      if (want_ddA) {
        part += __shfl_xor(part, 32);  // the halves of the wave hold different columns n of row m
        if (half == 0) rs[wave * 32 + l32] = part * w;
      }
    }
    __syncthreads();
    if (want_ddA && tid < 64) {
      // rows 32 * (tid / 32) .. belong to the waves w0 = tid / 32 and w0 + 2, which own different
      // columns of them
      const int w0 = tid >> 5;
      const float r = rs[w0 * 32 + (tid & 31)] + rs[(w0 + 2) * 32 + (tid & 31)];
      const int m = m0 + tid;
      float* o = ddA + chunk * Q;
      if (MODE == 0) {
        if (m + 1 < Q) o[m + 1] = r;
        if (m == 0) o[0] = 0.f;
      } else if (m < Q) {
        o[m] = r;
      }
    }
    // the next head's staging overwrites St; rs is rewritten only after the next barrier
  }
  // total is [n][m] per block: a lane writes four adjacent n of its row m at a time
  float* og = out + (b * L + (int64_t)c * Q) * ngroups * N + (int64_t)g * N;
  const int m = m0 + 32 * mi[0] + l32;
  if (m < limit) {
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; v += 4)
        *reinterpret_cast<float4*>(og + (int64_t)m * ngroups * N + 32 * ni[i] + acc_row(v, lane)) =
            make_float4(total[i][v], total[i][v + 1], total[i][v + 2], total[i][v + 3]);
  }
}

// ------------------------------------------------------------------------------------
// The same for bfloat16 operands and states, hdim 64, dstate 128, chunk sizes that are multiples of
// 64, no packed batch.  A workgroup spends most of a head waiting for the head's state tile and rows,
// and the registers do not hold a second head next to the accumulators, so here everything a head
// needs is copied from global memory straight into LDS by the load unit (no registers in between):
// three heads' worth of LDS, the copies of heads h + 1 and h + 2 under way while head h is
// multiplied, one barrier per head.  A copy puts the 16-byte pieces that the 64 lanes ask for side
// by side (1 KB per instruction), so the tiles have no padding; bank conflicts are avoided by
// the order of the pieces inside a row, which the requesting lane chooses through the address it
// asks for:
//   state tile [64 p][128 n] (256-byte rows, read with the transposing read): piece j of row r in slot
//     j ^ 4 (r % 4), so that four consecutive rows fall into four different quarters of the bank period;
//   rows of a [64 m][64 p] (128-byte rows, read 16 bytes per lane, a lane per row): piece j of row r in
//     slot j ^ ((r / 2) % 8), so that sixteen consecutive rows cover all banks;
//   one more instruction brings dA[m0 .. m0 + 63], dt[m0 .. m0 + 63] and dA[Q - 4 .. Q - 1].
// The copies count as vector-memory loads of the requesting wave and complete in order; a wave waits
// until only the copies of the head after the current one are outstanding, then passes the barrier.
// ------------------------------------------------------------------------------------
struct GroupDmaSmem {
  static constexpr int R = 3;  // heads in LDS
  static constexpr int kState = 64 * 128 * (int)sizeof(bf16_t), kRows = 64 * 64 * (int)sizeof(bf16_t), kVec = 2048;
  static constexpr int kHead = kState + kRows + kVec;
  static constexpr int kBytes = R * kHead + 2 * 4 * 32 * (int)sizeof(float);  // + the row sums of two heads
  // copies a wave requests per head (the first wave one more: the vectors)
  static constexpr int kCopiesPerWave = 16 / 4 + 8 / 4;
};

template <int MODE>
__global__ __launch_bounds__(256, 2) void ssd_group_grad_dma_kernel(
    const bf16_t* __restrict__ a, Strides3 sa, const bf16_t* __restrict__ s, const float* __restrict__ dt,
    const float* __restrict__ dA_cs, const bf16_t* __restrict__ bc, Strides3 sbc, float* __restrict__ out,
    float* __restrict__ ddA, int nh, int heads_per_group, int ngroups, int L, int Q, int C, int mtiles) {
  using S = GroupDmaSmem;
  using T = bf16_t;
  constexpr int P = 64, N = 128, EPL = 8, KG = 16, BPW = 2, KS = P / KG;
  static_assert(S::kCopiesPerWave == 6, "the wait below counts six copies per wave and head");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* rs = reinterpret_cast<float*>(smem + S::R * S::kHead);  // [2 heads][4 waves][32 rows]

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int mt = bid % mtiles;
  const int g = (bid / mtiles) % ngroups;
  const int c = (bid / (mtiles * ngroups)) % C;
  const int64_t b = bid / ((int64_t)mtiles * ngroups * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = 64 * mt;

  // block i of this wave: rows 32 * mi .., columns 32 * ni[i] ..
  const int mi = wave & 1;
  int ni[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) ni[i] = (wave + 4 * i) >> 1;
  const int rloc = 32 * mi + l32;  // this lane's row inside the tile
  const int m = m0 + rloc;
  const bool want_ddA = bc != nullptr;
  floatx16 total[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) zero_acc(total[i]);

  // The copies of head hh into LDS set u.  What depends on the lane is the same for every head and is
  // kept as byte offsets; a head only moves the (scalar) bases.
  // Copies a wave requests per head: kSCopies of the state tile, kACopies of the rows (and one more on
  // waves 0 / 1); the wait in the loop counts on these numbers.
  constexpr int kSCopies = 4, kACopies = 2, kMinCopies = kSCopies + kACopies;
  static_assert(4 * 4 * kSCopies == P && 4 * 8 * kACopies == 64, "four waves bring a head's state tile and 64 rows");
  unsigned s_off[kSCopies], a_off[kACopies];
#pragma unroll
  for (int j = 0; j < kSCopies; ++j) {  // four rows of the state tile per instruction
    const int r = 4 * (4 * wave + j) + (lane >> 4);
    s_off[j] = (unsigned)(r * N + 8 * ((lane & 15) ^ (4 * (r & 3)))) * (unsigned)sizeof(T);
  }
#pragma unroll
  for (int j = 0; j < kACopies; ++j) {  // eight rows of a per instruction
    const int r = 8 * (2 * wave + j) + (lane >> 3);
    a_off[j] = (unsigned)((int64_t)min(m0 + r, limit - 1) * sa.sl + 8 * ((lane & 7) ^ ((r >> 1) & 7))) * (unsigned)sizeof(T);
  }
  // waves 0 and 1 bring dA[m0 .. m0 + 63] with dA[Q - 4 .. Q - 1] behind it, and dt[m0 .. m0 + 63]
  const unsigned v_off = (unsigned)(lane < 16 ? m0 + 4 * lane : (wave == 0 ? Q - 4 : m0)) * (unsigned)sizeof(float);
  const T* s_first = s + (((b * C + c) * nh + g * heads_per_group) * (int64_t)P) * N;
  const T* a_first = a + b * sa.sb + (int64_t)c * Q * sa.sl + (int64_t)g * heads_per_group * sa.sh;
  const int64_t chunk_first = (b * nh + g * heads_per_group) * (int64_t)C + c;
  auto request = [&](int hh, int u) {
    unsigned char* base = smem + u * S::kHead;
    const T* sg = s_first + (int64_t)hh * P * N;
    const T* ag = a_first + (int64_t)hh * sa.sh;
#pragma unroll
    for (int j = 0; j < kSCopies; ++j) copy16_to_lds(sg, s_off[j], base + (4 * wave + j) * 1024);
#pragma unroll
    for (int j = 0; j < kACopies; ++j) copy16_to_lds(ag, a_off[j], base + S::kState + (2 * wave + j) * 1024);
    if (wave < 2) {
      const float* vg = (wave == 0 ? dA_cs : dt) + (chunk_first + (int64_t)hh * C) * Q;
      copy16_to_lds(vg, v_off, base + S::kState + S::kRows + wave * 1024);
    }
  };
  request(0, 0);
  if (heads_per_group > 1) request(1, 1);
  // bc in the (transposed) accumulator layout: this lane's row m, columns n of each block.  Loaded
  // behind the first copies and waited for here, so that no wait for ordinary loads (which would wait
  // for every copy before them as well) falls into the loop.
  float bcv[BPW][16];
#pragma unroll
  for (int i = 0; i < BPW; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) bcv[i][v] = 0.f;
  if (want_ddA) {
    const T* bcg = bc + b * sbc.sb + (int64_t)c * Q * sbc.sl + g * sbc.sh;
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float t = (float)bcg[(int64_t)min(m, limit - 1) * sbc.sl + 32 * ni[i] + acc_row(v, lane)];
        bcv[i][v] = m < limit ? t : 0.f;
      }
  }
#pragma unroll
  for (int i = 0; i < BPW; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(bcv[i][v]));

  // where this lane reads its operand fragments inside a head's tiles (elements)
  int r_off[KS], t_off[BPW];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) r_off[ks] = rloc * P + 8 * ((2 * ks + half) ^ ((rloc >> 1) & 7));
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int i16 = lane & 15;
    const int row = 8 * half + (i16 >> 2);
    const int col = 32 * ni[i] + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    t_off[i] = row * N + 8 * ((col >> 3) ^ (4 * (row & 3))) + (col & 7);
  }

  for (int hh = 0; hh < heads_per_group; ++hh) {
    const int u = hh % S::R;
    // the copies of this head have landed once only those of the next head are outstanding
    if (hh + 1 < heads_per_group) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kMinCopies) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // every wave's part of the head is there; every wave is done with head hh - 1
    if (hh + 2 < heads_per_group) request(hh + 2, (hh + 2) % S::R);
    if (want_ddA && hh > 0 && tid < 64) {  // the row sums of head hh - 1 (see below)
      const float* rp = rs + ((hh - 1) & 1) * 128;
      const int w0 = tid >> 5;
      const float r = rp[w0 * 32 + (tid & 31)] + rp[(w0 + 2) * 32 + (tid & 31)];
      float* o = ddA + ((b * nh + g * heads_per_group + hh - 1) * C + c) * (int64_t)Q;
      const int mm = m0 + tid;
      if (MODE == 0) {
        if (mm + 1 < Q) o[mm + 1] = r;
        if (mm == 0) o[0] = 0.f;
      } else {
        o[mm] = r;
      }
    }
    const unsigned char* base = smem + u * S::kHead;
    const T* St = reinterpret_cast<const T*>(base);
    const T* At = reinterpret_cast<const T*>(base + S::kState);
    const float* vec = reinterpret_cast<const float*>(base + S::kState + S::kRows);  // dA rows, dA tail | dt rows
    // the weight of this lane's row; rows past the sequence (their operand rows repeat the last
    // valid one) get none
    const float wr = MODE == 0 ? __expf(fminf(vec[67] - vec[rloc], 0.f)) * vec[256 + rloc] : __expf(vec[rloc]);
    const float w = m < limit ? wr : 0.f;
    floatx16 acc[BPW];
#pragma unroll
    for (int i = 0; i < BPW; ++i) zero_acc(acc[i]);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const Vec16<T> av = load16(At + r_off[ks]);
#pragma unroll
      for (int i = 0; i < BPW; ++i) {
        // St[p][n] contracted along p: lane l receives eight consecutive p of column n = 32 ni + l % 32
        // (sixteen rows further down the key of a row is the same)
        const T* p = St + t_off[i] + KG * ks * N;
        typedef __attribute__((address_space(3))) ema::bf16x4 lds_bf16x4;
        const ema::bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
        const ema::bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * N));  // row + 4: the same key
        Vec16<T> sf;
        sf.raw = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        mma_group(sf, av, acc[i]);  // [n][m]
      }
    }
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        total[i][v] = fmaf(acc[i][v], w, total[i][v]);
        part = fmaf(acc[i][v], bcv[i][v], part);  // bcv is zero where no row sums are asked for
      }
    if (want_ddA) {
      // the halves of the wave hold different columns n of row m; the waves w and w + 2 too: their
      // sums meet after the next barrier
      part += __shfl_xor(part, 32);
      if (half == 0) rs[(hh & 1) * 128 + wave * 32 + l32] = part * w;
    }
  }
  if (want_ddA) {
    __syncthreads();
    if (tid < 64) {
      const int hh = heads_per_group - 1;
      const float* rp = rs + (hh & 1) * 128;
      const int w0 = tid >> 5;
      const float r = rp[w0 * 32 + (tid & 31)] + rp[(w0 + 2) * 32 + (tid & 31)];
      float* o = ddA + ((b * nh + g * heads_per_group + hh) * C + c) * (int64_t)Q;
      const int mm = m0 + tid;
      if (MODE == 0) {
        if (mm + 1 < Q) o[mm + 1] = r;
        if (mm == 0) o[0] = 0.f;
      } else {
        o[mm] = r;
      }
    }
  }
  // total is [n][m] per block: a lane writes four adjacent n of its row m at a time
  float* og = out + (b * L + (int64_t)c * Q) * ngroups * N + (int64_t)g * N;
  if (m < limit) {
#pragma unroll
    for (int i = 0; i < BPW; ++i)
#pragma unroll
      for (int v = 0; v < 16; v += 4)
        *reinterpret_cast<float4*>(og + (int64_t)m * ngroups * N + 32 * ni[i] + acc_row(v, lane)) =
            make_float4(total[i][v], total[i][v + 1], total[i][v + 2], total[i][v + 3]);
  }
}

// ------------------------------------------------------------------------------------
// bmm_chunk.  out[b, c, g, m, k] = sum_n a[b, cQ+m, g, n] * bm[b, cQ+k, g, n]; one workgroup
// per 64 x 64 output tile, one 32 x 32 block per wave; rows past the sequence are zero, and so
// are, in a packed batch, the entries whose two positions carry different ids.
// ------------------------------------------------------------------------------------
template <typename T, int K>
constexpr int bmm_smem_bytes() {
  return 2 * 64 * Tile<T>::pitch(K) * (int)sizeof(T);
}

template <typename T, typename TO, int K>
__global__ __launch_bounds__(256) void ssd_bmm_kernel(const T* __restrict__ a, Strides3 sa,
                                                      const T* __restrict__ bm, Strides3 sb_,
                                                      TO* __restrict__ out, int ngroups, int L, int Q, int C,
                                                      int tiles, SeqIdx seq) {
  constexpr int PK = Tile<T>::pitch(K), KG = Tile<T>::KG;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* as = reinterpret_cast<T*>(smem);
  T* bs = as + 64 * PK;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int tn = bid % tiles;
  const int tm = (bid / tiles) % tiles;
  const int64_t bcg = bid / (tiles * tiles);
  const int g = (int)(bcg % ngroups);
  const int c = (int)((bcg / ngroups) % C);
  const int64_t b = bcg / ((int64_t)ngroups * C);
  const int limit = min(Q, L - c * Q);
  stage_rows<T, 64, K>(as, a + b * sa.sb + (int64_t)c * Q * sa.sl + g * sa.sh, sa.sl, 64 * tm, limit, tid, NoScale());
  stage_rows<T, 64, K>(bs, bm + b * sb_.sb + (int64_t)c * Q * sb_.sl + g * sb_.sh, sb_.sl, 64 * tn, limit, tid,
                       NoScale());
  __syncthreads();
  const int wm = wave >> 1, wn = wave & 1;
  floatx16 acc;
  zero_acc(acc);
#pragma unroll
  for (int kk = 0; kk < K; kk += KG)
    mma_group(frag_rows(as, PK, 32 * wm, kk, lane), frag_rows(bs, PK, 32 * wn, kk, lane), acc);
  TO* o = out + bcg * (int64_t)Q * Q;
  const int col = 64 * tn + 32 * wn + (lane & 31);
  const ChunkSeq sq = chunk_seq(seq, b, c, Q);
  const int col_id = sq.on() ? sq.at(min(col, limit - 1)) : 0;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = 64 * tm + 32 * wm + acc_row(v, lane);
    float val = acc[v];
    if (sq.on() && sq.at(min(row, limit - 1)) != col_id) val = 0.f;
    if (row < Q && col < Q) o[(int64_t)row * Q + col] = (TO)val;
  }
}

// ------------------------------------------------------------------------------------
// chunk_scan.  One workgroup per (b, c, h, tile of 64 rows m):
//   out[m][p] = exp(dA_m) * sum_n C[m][n] * round_T(prev[p][n])
//             + sum_{k <= m} round_T(cb[m][k] * exp(min(dA_m - dA_k, 0)) * dt_k) * x[k][p]
//             + D * x[m][p],            then out_x = out (if asked) and out *= z * sigmoid(z).
// The causal sum walks the 64-row tiles k up to the diagonal one; the result leaves through an
// LDS tile so that z, out and out_x move in 16-byte pieces.  In a packed batch the carried state
// only reaches the rows whose id equals that of the previous chunk's last position (cb already
// holds zeros between positions of different ids).
// cb is float32 (b, C, g, Q, Q); prev is (b, C, nh, P, N) in float32 or in T (type TS).
// ------------------------------------------------------------------------------------
template <typename T, int P, int N>
struct ScanSmem {
  static constexpr int PC = Tile<T>::pitch(N), PX = Tile<T>::pitch(P), PW = Tile<T>::pitch(64), PO = P + 4;
  static constexpr int kPhaseA = (64 + P) * PC * (int)sizeof(T);                 // C tile, prev tile
  static constexpr int kPhaseB = (64 * PX + 64 * PW) * (int)sizeof(T);           // x tile, weights
  static constexpr int kPhaseC = 64 * PO * (int)sizeof(float);                   // output staging
  static constexpr int kMax1 = kPhaseA > kPhaseB ? kPhaseA : kPhaseB;
  static constexpr int kBytes = (kMax1 > kPhaseC ? kMax1 : kPhaseC) + 64 * (int)sizeof(float);
};

template <typename T, int P, int N, typename TS>
__global__ __launch_bounds__(256) void ssd_chunk_scan_kernel(
    const float* __restrict__ cb, const T* __restrict__ x, Strides3 sx, const T* __restrict__ z, Strides3 sz,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, const T* __restrict__ Cm, Strides3 sC,
    const TS* __restrict__ prev, const float* __restrict__ D, int d_has_hdim, T* __restrict__ out,
    Strides3 so, T* __restrict__ out_x, int nh, int heads_per_group, int ngroups, int L, int Q, int C,
    int mtiles, SeqIdx seq) {
  using S = ScanSmem<T, P, N>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, PB = P / 32, BPW = 2 * PB / 4;
  static_assert(PB == 2 || PB == 4, "hdim 64 or 128");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Cs = reinterpret_cast<T*>(smem);
  T* Ps = Cs + 64 * S::PC;
  T* Xs = reinterpret_cast<T*>(smem);
  T* Ws = Xs + 64 * S::PX;
  float* Os = reinterpret_cast<float*>(smem);
  float* sm = reinterpret_cast<float*>(smem + S::kBytes - 64 * sizeof(float));  // exp(dA_m)

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int mt = bid % mtiles;
  const int h = (bid / mtiles) % nh;
  const int c = (bid / (mtiles * nh)) % C;
  const int64_t b = bid / ((int64_t)mtiles * nh * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = 64 * mt;
  if (m0 >= limit) return;
  const int g = h / heads_per_group;
  const int64_t chunk = (b * nh + h) * C + c;
  const float* dAp = dA_cs + chunk * Q;
  const float* dtp = dt + chunk * Q;
  const T* xg = x + b * sx.sb + (int64_t)c * Q * sx.sl + h * sx.sh;
  const T* Cg = Cm + b * sC.sb + (int64_t)c * Q * sC.sl + g * sC.sh;
  const TS* pg = prev + (((b * C + c) * nh + h) * (int64_t)P) * N;
  const float* cbg = cb + (((b * C + c) * ngroups + g) * (int64_t)Q) * Q;

  // wave -> output blocks: rows 32*mi.., columns 32*(pi0 + 2*i)..
  const int mi = wave & 1, pi0 = wave >> 1;
  floatx16 acc[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) zero_acc(acc[i]);

  // ---- phase A: C . prev, scaled by exp(dA_m)
  stage_rows<T, 64, N>(Cs, Cg, sC.sl, m0, limit, tid, NoScale());
  {
    constexpr int VPR = N / 4;  // float4 per row of prev
#pragma unroll
    for (int i = 0; i < P * VPR / 256; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / VPR, cv = (idx % VPR) * 4;
      const float4 v = state_load4<false>(pg + (int64_t)r * N + cv);
      T* d = Ps + r * S::PC + cv;
      d[0] = (T)v.x, d[1] = (T)v.y, d[2] = (T)v.z, d[3] = (T)v.w;
    }
  }
  if (tid < 64) {
    const ChunkSeq sq = chunk_seq(seq, b, c, Q);
    const bool live = !sq.on() || sq.at(min(m0 + tid, limit - 1)) == sq.entering(c);
    sm[tid] = (m0 + tid < Q && live) ? __expf(dAp[m0 + tid]) : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int kk = 0; kk < N; kk += KG) {
    const Vec16<T> a = frag_rows(Cs, S::PC, 32 * mi, kk, lane);
#pragma unroll
    for (int i = 0; i < BPW; ++i) mma_group(a, frag_rows(Ps, S::PC, 32 * (pi0 + 2 * i), kk, lane), acc[i]);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float s = sm[32 * mi + acc_row(v, lane)];
#pragma unroll
    for (int i = 0; i < BPW; ++i) acc[i][v] *= s;
  }
  __syncthreads();

  // ---- phase B: causal sum over the k tiles up to the diagonal one
  for (int kt = 0; kt <= mt; ++kt) {
    const int k0 = 64 * kt;
    stage_rows<T, 64, P>(Xs, xg, sx.sl, k0, limit, tid, NoScale());
    {
      // weights: 64 x 64 float32 of cb -> scaled, masked, rounded to T; 16 float4 per row
#pragma unroll
      for (int i = 0; i < 64 * 16 / 256; ++i) {
        const int idx = tid + 256 * i;
        const int r = idx >> 4, cv = (idx & 15) * 4;
        const int m = m0 + r;
        T* d = Ws + r * S::PW + cv;
        // unconditional loads from indices clamped into the chunk (Q is a multiple of 4)
        const bool in = m < Q && k0 + cv < Q;
        const int mc = min(m, Q - 1), kc = min(k0 + cv, Q - 4);
        const float4 w4 = *reinterpret_cast<const float4*>(cbg + (int64_t)mc * Q + kc);
        const float4 a4 = *reinterpret_cast<const float4*>(dAp + kc);
        const float4 t4 = *reinterpret_cast<const float4*>(dtp + kc);
        const float am = dAp[mc];
        const float w[4] = {w4.x, w4.y, w4.z, w4.w}, ak[4] = {a4.x, a4.y, a4.z, a4.w},
                    tk[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          d[e] = (T)((in && k0 + cv + e <= m) ? w[e] * __expf(fminf(am - ak[e], 0.f)) * tk[e] : 0.f);
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 64; kk += KG) {
      const Vec16<T> a = frag_rows(Ws, S::PW, 32 * mi, kk, lane);
#pragma unroll
      for (int i = 0; i < BPW; ++i) mma_group(a, frag_cols(Xs, S::PX, kk, 32 * (pi0 + 2 * i), lane), acc[i]);
    }
    if (kt == mt && D) {  // the diagonal tile holds rows m0.. of x: the skip term
#pragma unroll
      for (int i = 0; i < BPW; ++i) {
        const int col = 32 * (pi0 + 2 * i) + (lane & 31);
        const float dv = d_has_hdim ? D[h * P + col] : D[h];
#pragma unroll
        for (int v = 0; v < 16; ++v)
          acc[i][v] = fmaf(dv, (float)Xs[(32 * mi + acc_row(v, lane)) * S::PX + col], acc[i][v]);
      }
    }
    __syncthreads();
  }

  // ---- phase C: through LDS to global memory, gate on the way
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int col = 32 * (pi0 + 2 * i) + (lane & 31);
#pragma unroll
    for (int v = 0; v < 16; ++v) Os[(32 * mi + acc_row(v, lane)) * S::PO + col] = acc[i][v];
  }
  __syncthreads();
  constexpr int VPR = P / EPL;
#pragma unroll
  for (int i = 0; i < 64 * VPR / 256; ++i) {
    const int idx = tid + 256 * i;
    const int r = idx / VPR, cv = (idx % VPR) * EPL;
    const int m = m0 + r;
    if (m >= limit) continue;
    const int64_t pos = (int64_t)c * Q + m;
    float v[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = Os[r * S::PO + cv + e];
    Vec16<T> o;
    if (z) {
      if (out_x) {
        o.set_all(v);
        store16(out_x + b * so.sb + pos * so.sl + h * so.sh + cv, o);
      }
      const Vec16<T> zv = load16(z + b * sz.sb + pos * sz.sl + h * sz.sh + cv);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const float zf = zv.get(e);
        v[e] *= zf / (1.f + __expf(-zf));
      }
    }
    o.set_all(v);
    store16(out + b * so.sb + pos * so.sl + h * so.sh + cv, o);
  }
}

// ------------------------------------------------------------------------------------
// chunk_scan for chunk sizes that are multiples of 256.  One workgroup per (b, c, h, 256-row
// super-tile); wave w owns the 32-row blocks w and 7 - w of it, which balances the causal sum,
// and all hdim / 32 column blocks.  The operands that differ from lane to lane are built in
// registers straight from global memory (C rows; cb rows, weighted and masked on the way), so
// the k loop has no barrier: LDS only holds what every wave shares, the 256-row tile of x, the
// carried state and the chunk's dA / dt.  Results leave through a per-wave LDS staging area.
// ------------------------------------------------------------------------------------
template <typename T, int P, int N>
struct WideSmem {
  static constexpr int ST = 256;
  static constexpr int PX = Tile<T>::pitch(P), PC = Tile<T>::pitch(N), PO = P + 4;
  static constexpr int kX = ST * PX * (int)sizeof(T);
  static constexpr int kPrev = P * PC * (int)sizeof(T);
  static constexpr int kOut = 4 * 32 * PO * (int)sizeof(float);                  // one 32-row block per wave
  // the carried state is only read before the k loop, the x tile only inside it, the output
  // staging only after it: the three share one region
  static constexpr int kXP = kX > kPrev ? kX : kPrev;
  static constexpr int kMain = kXP > kOut ? kXP : kOut;
  static constexpr int kBytes = kMain + 3 * ST * (int)sizeof(float);            // + dA_k, dt_k, exp(dA_m)
  // the same with those three vectors for each of `heads` heads sharing a tile of this width
  static constexpr int bytes_for(int heads) { return kMain + heads * 3 * ST * (int)sizeof(float); }
};

// HP heads per workgroup (1 or 2).  Two adjacent heads of one group share everything that does not
// depend on the head: the fragments of cb and the rows of C, which are the costly per-lane loads of
// this kernel.  Their x / z / out rows and their carried states are adjacent in memory (heads are
// dense in those tensors; the host checks), so the pair is staged and stored like one head of twice
// the width; the weights, the scale of the carried-state term and D are per head.
template <typename T, int P, int N, typename TS, int HP>
__global__ __launch_bounds__(256, 2) void ssd_chunk_scan_wide_kernel(
    const float* __restrict__ cb, const T* __restrict__ x, Strides3 sx, const T* __restrict__ z, Strides3 sz,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, const T* __restrict__ Cm, Strides3 sC,
    const TS* __restrict__ prev, const float* __restrict__ D, int d_has_hdim, T* __restrict__ out,
    Strides3 so, T* __restrict__ out_x, int nh, int heads_per_group, int ngroups, int L, int Q, int C,
    int stiles, SeqIdx seq) {
  constexpr int PW = P * HP;  // width of the tile of x, z and out
  using S = WideSmem<T, PW, N>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, PB = PW / 32, PBH = P / 32, ST = S::ST;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Xs = reinterpret_cast<T*>(smem);
  T* Pv = reinterpret_cast<T*>(smem);
  float* Os = reinterpret_cast<float*>(smem);
  float* vec = reinterpret_cast<float*>(smem + S::kMain);  // per head: dA_k, dt_k, exp(dA_m) / factor
  auto dAk = [&](int hh) { return vec + (3 * hh) * ST; };
  auto dtk = [&](int hh) { return vec + (3 * hh + 1) * ST; };
  auto sm = [&](int hh) { return vec + (3 * hh + 2) * ST; };  // exp(dA_m) of the carried-state term, then
  auto fk = [&](int hh) { return vec + (3 * hh + 2) * ST; };  // the per-position factor of the causal term

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int nhp = nh / HP;
  const int st = bid % stiles;
  const int h = ((bid / stiles) % nhp) * HP;  // first head of the workgroup
  const int c = (bid / (stiles * nhp)) % C;
  const int64_t b = bid / ((int64_t)stiles * nhp * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = ST * st;
  if (m0 >= limit) return;
  const int g = h / heads_per_group;
  const float* dAp[HP];
  const float* dtp[HP];
#pragma unroll
  for (int hh = 0; hh < HP; ++hh) {
    const int64_t chunk = (b * nh + h + hh) * C + c;
    dAp[hh] = dA_cs + chunk * Q;
    dtp[hh] = dt + chunk * Q;
  }
  const T* xg = x + b * sx.sb + (int64_t)c * Q * sx.sl + h * sx.sh;
  const T* Cg = Cm + b * sC.sb + (int64_t)c * Q * sC.sl + g * sC.sh;
  const TS* pg = prev + (((b * C + c) * nh + h) * (int64_t)P) * N;
  const float* cbg = cb + (((b * C + c) * ngroups + g) * (int64_t)Q) * Q;

  int mrow[2];
  mrow[0] = 32 * wave;
  mrow[1] = 32 * (7 - wave);
  floatx16 acc[2][PB];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) zero_acc(acc[mb][pb]);

  SSD_TSTAMP(0);
  // The carried state only takes the lower half of the region it shares with the x tile: the upper half
  // of the first x tile, rows 128 .. 255, is requested now, ahead of the state, and written to LDS behind
  // it, so that it costs no round trip of its own after phase A.
  static_assert(S::kPrev <= (ST / 2) * S::PX * (int)sizeof(T), "the carried state must leave the upper half of the x tile free");
  constexpr bool kEarly = (ST / 2) * (PW / EPL) / 256 <= 8;  // (eight pieces per thread travel in registers)
  RowPieces<T, kEarly ? ST / 2 : 32, kEarly ? PW : EPL * 8, S::PX> upper;
  if constexpr (kEarly) upper.template load<true>(xg, sx.sl, ST / 2, limit, tid);
  // ---- phase A: C . prev, scaled by exp(dA_m)
  {
    constexpr int VPR = N / 4;
#pragma unroll
    for (int i = 0; i < PW * VPR / 256; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / VPR, cv = (idx % VPR) * 4;
      const float4 v = state_load4<true>(pg + (int64_t)r * N + cv);
      T* d = Pv + r * S::PC + cv;
      d[0] = (T)v.x, d[1] = (T)v.y, d[2] = (T)v.z, d[3] = (T)v.w;
    }
  }
  {
    const ChunkSeq sq = chunk_seq(seq, b, c, Q);
    const bool live = !sq.on() || sq.at(min(m0 + tid, limit - 1)) == sq.entering(c);
#pragma unroll
    for (int hh = 0; hh < HP; ++hh) sm(hh)[tid] = live ? __expf(dAp[hh][m0 + tid]) : 0.f;
  }
  if constexpr (kEarly) upper.store(Xs + (ST / 2) * S::PX, ST / 2, limit, tid, NoScale());
  __syncthreads();
  SSD_TSTAMP(1);
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int m = m0 + mrow[mb] + l32;
    const T* crow = Cg + (int64_t)min(m, limit - 1) * sC.sl + EPL * half;
#pragma unroll
    for (int kk = 0; kk < N; kk += KG) {
      Vec16<T> a = load16(crow + kk);  // row clamped into the sequence, zeroed if past it
      if (m >= limit) a.zero();
#pragma unroll
      for (int pb = 0; pb < PB; ++pb) mma_group(a, frag_rows(Pv, S::PC, 32 * pb, kk, lane), acc[mb][pb]);
    }
#pragma unroll
    for (int hh = 0; hh < HP; ++hh)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float sc = sm(hh)[mrow[mb] + acc_row(v, lane)];
#pragma unroll
        for (int pb = hh * PBH; pb < (hh + 1) * PBH; ++pb) acc[mb][pb][v] *= sc;
      }
  }

  // ---- phase B: the k super-tiles up to the diagonal one
  SSD_TSTAMP(2);
  __syncthreads();  // the x tile takes the place of the carried state
  SSD_TSTAMP(3);
  for (int kt = 0; kt <= st; ++kt) {
    const int k0 = ST * kt;
    // (the upper half of the first tile is in LDS already, see above)
    stage_rows<T, ST / 2, PW, NoScale, true>(Xs, xg, sx.sl, k0, limit, tid, NoScale());
    if (kt > 0 || !kEarly) stage_rows<T, ST / 2, PW, NoScale, true>(Xs + (ST / 2) * S::PX, xg, sx.sl, k0 + ST / 2, limit, tid, NoScale());
#pragma unroll
    for (int hh = 0; hh < HP; ++hh) {
      // Below the diagonal the weight of (m, k) is split at the last position r of k's group of
      // 32: exp(dA_m - dA_r) is one exponential per row and group, exp(dA_r - dA_k) * dt_k one
      // per position k, shared by all rows.  Each exponent is clamped at 0 like the whole is in
      // the reference; for a dA_cumsum that is monotone inside the chunk (A of one sign,
      // dt >= 0) the product is the reference's clamped exponential.
      const float ak = dAp[hh][k0 + tid], ar = dAp[hh][k0 + (tid | 31)], tk = dtp[hh][k0 + tid];
      dAk(hh)[tid] = ak;
      dtk(hh)[tid] = tk;
      fk(hh)[tid] = __expf(fminf(ar - ak, 0.f)) * tk;
    }
    __syncthreads();
    SSD_TSTAMP(4);
    const bool diag = kt == st;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int mloc = mrow[mb] + l32;  // row inside the super-tile
      float am[HP];
#pragma unroll
      for (int hh = 0; hh < HP; ++hh) am[hh] = dAp[hh][m0 + mloc];
      const float* cbrow = cbg + (int64_t)(m0 + mloc) * Q + k0 + EPL * half;
      const int kend = diag ? mrow[mb] + 32 : ST;
      // NS steps at a time (the step count is even): their cb fragments are all requested before
      // the first is used, so the wave waits for memory once per NS steps.  Only where the
      // registers allow it without losing a wave per SIMD.
      constexpr int NS = (PW == 64 && sizeof(T) == 2) ? 2 : 1;
      for (int kk0 = 0; kk0 < kend; kk0 += NS * KG) {
        float w[NS][EPL];
#pragma unroll
        for (int u = 0; u < NS; ++u)
#pragma unroll
          for (int e = 0; e < EPL; e += 4) {
            const float4 c4 = *reinterpret_cast<const float4*>(cbrow + kk0 + KG * u + e);
            w[u][e] = c4.x, w[u][e + 1] = c4.y, w[u][e + 2] = c4.z, w[u][e + 3] = c4.w;
          }
        // the group of 32 positions that holds the diagonal takes the exact, masked form
        const int grp_last = (kk0 & ~31) + 31;
        const bool exact = diag && grp_last >= mrow[mb];
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
          const float gm = __expf(fminf(am[hh] - dAk(hh)[grp_last], 0.f));
#pragma unroll
          for (int u = 0; u < NS; ++u) {
            const int kk = kk0 + KG * u, kb = kk + EPL * half;
            Vec16<T> a;
            float wf[EPL];
            if (exact) {
#pragma unroll
              for (int e = 0; e < EPL; ++e) {
                const float f = w[u][e] * __expf(fminf(am[hh] - dAk(hh)[kb + e], 0.f)) * dtk(hh)[kb + e];
                wf[e] = kb + e > mloc ? 0.f : f;
              }
            } else {
#pragma unroll
              for (int e = 0; e < EPL; ++e) wf[e] = w[u][e] * fk(hh)[kb + e] * gm;
            }
            a.set_all(wf);
#pragma unroll
            for (int pb = hh * PBH; pb < (hh + 1) * PBH; ++pb)
              mma_group(a, frag_cols(Xs, S::PX, kk, 32 * pb, lane), acc[mb][pb]);
          }
        }
      }
      if (diag && D) {
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
          const int col = 32 * pb + l32;  // column of the tile = feature of head h + col / P
          const float dv = d_has_hdim ? D[h * P + col] : D[h + pb / PBH];
#pragma unroll
          for (int v = 0; v < 16; ++v)
            acc[mb][pb][v] = fmaf(dv, (float)Xs[(mrow[mb] + acc_row(v, lane)) * S::PX + col], acc[mb][pb][v]);
        }
      }
    }
    SSD_TSTAMP(5);
    __syncthreads();
  }
  SSD_TSTAMP(6);

  // ---- phase C: each wave moves its two blocks through its own staging area
  float* mine = Os + wave * 32 * S::PO;
  constexpr int VPR = PW / EPL;
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
    for (int pb = 0; pb < PB; ++pb)
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[acc_row(v, lane) * S::PO + 32 * pb + l32] = acc[mb][pb][v];
    // the wave's own writes are visible to its own reads once the LDS counter has drained
    __builtin_amdgcn_s_waitcnt(0xc07f);
#pragma unroll
    for (int i = 0; i < 32 * VPR / 64; ++i) {
      const int idx = lane + 64 * i;
      const int r = idx / VPR, cv = (idx % VPR) * EPL;
      const int m = m0 + mrow[mb] + r;
      if (m < limit) {
        const int64_t pos = (int64_t)c * Q + m;
        float v[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) v[e] = mine[r * S::PO + cv + e];
        Vec16<T> o;
        if (z) {
          if (out_x) {
            o.set_all(v);
            store16(out_x + b * so.sb + pos * so.sl + h * so.sh + cv, o);
          }
          const Vec16<T> zv = load16(z + b * sz.sb + pos * sz.sl + h * sz.sh + cv);
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            const float zf = zv.get(e);
            v[e] *= zf / (1.f + __expf(-zf));
          }
        }
        o.set_all(v);
        store16_stream(out + b * so.sb + pos * so.sl + h * so.sh + cv, o);
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  SSD_TSTAMP(7);
}

// Partial sums for the gradient of the skip weight D: a lane holds, for its EPL adjacent features
// cv .. (cv = EPL * (lane % VPR)), the sum of dout * x over the rows it handled; the lanes of a
// wave that share cv are added up and the wave's hdim sums go to its slot.  The caller adds the
// slots of all waves, chunks and batch elements.
template <int EPL, int VPR>
__device__ __forceinline__ void store_dD_partial(float* __restrict__ slot, float* dsum, int lane) {
#pragma unroll
  for (int off = VPR; off < 64; off <<= 1)
#pragma unroll
    for (int e = 0; e < EPL; ++e) dsum[e] += __shfl_xor(dsum[e], off);
  if (lane < VPR) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) slot[lane * EPL + e] = dsum[e];
  }
}

// ------------------------------------------------------------------------------------
// Backward of chunk_scan and chunk_state with respect to x (and the explicit dt factors).
// One workgroup per (b, c, h, tile of 64 rows m):
//   acc[m][p] = exp(min(dA_last - dA_m, 0)) * sum_n B[m][n] * round_T(dstates[p][n])
//             + sum_{k >= m, k < limit} round_T(cb[k][m] * exp(min(dA_k - dA_m, 0))) * dout[k][p]
//   dx[m][p] = acc * dt_m + D * dout[m][p],    ddt[m] = sum_p acc[m][p] * x[m][p]
// The mirror image of ssd_chunk_scan_kernel: the k tiles run from the diagonal one to the end
// of the chunk, and the weights are staged transposed (k-major), so that cb is still read along
// its rows.  In a packed batch the dstates term only reaches the rows whose id equals that of the
// chunk's last position.
// ------------------------------------------------------------------------------------
template <typename T, int P, int N, typename TS>
__global__ __launch_bounds__(256) void ssd_chunk_scan_bwd_dx_kernel(
    const float* __restrict__ cb, const T* __restrict__ x, Strides3 sx, const T* __restrict__ dout, Strides3 sd,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, const T* __restrict__ Bm, Strides3 sB,
    const TS* __restrict__ dstates, const float* __restrict__ D, int d_has_hdim, T* __restrict__ dx,
    Strides3 sdx, float* __restrict__ ddt, int nh, int heads_per_group, int ngroups, int L, int Q, int C,
    int mtiles, SeqIdx seq, float* __restrict__ dD_part) {
  using S = ScanSmem<T, P, N>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, PB = P / 32, BPW = 2 * PB / 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Bs = reinterpret_cast<T*>(smem);
  T* Ps = Bs + 64 * S::PC;
  T* Ds = reinterpret_cast<T*>(smem);
  T* Wt = Ds + 64 * S::PX;  // [k][m]
  float* Os = reinterpret_cast<float*>(smem);
  float* sm = reinterpret_cast<float*>(smem + S::kBytes - 64 * sizeof(float));

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int mt = bid % mtiles;
  const int h = (bid / mtiles) % nh;
  const int c = (bid / (mtiles * nh)) % C;
  const int64_t b = bid / ((int64_t)mtiles * nh * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = 64 * mt;
  const int64_t chunk = (b * nh + h) * C + c;
  float* ddtp = ddt + chunk * Q;
  // slot of this wave in dD_part (batch, C, nheads, 4 * mtiles, hdim)
  float* dslot = dD_part ? dD_part + ((((b * C + c) * nh + h) * (int64_t)mtiles + mt) * 4 + wave) * P : nullptr;
  if (m0 >= limit) {  // nothing of the sequence in this tile: its ddt and dD slots are zero
    if (tid < 64 && m0 + tid < Q) ddtp[m0 + tid] = 0.f;
    if (dslot && lane < P / EPL) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) dslot[lane * EPL + e] = 0.f;
    }
    return;
  }
  const int g = h / heads_per_group;
  const float* dAp = dA_cs + chunk * Q;
  const float* dtp = dt + chunk * Q;
  const T* xg = x + b * sx.sb + (int64_t)c * Q * sx.sl + h * sx.sh;
  const T* dg = dout + b * sd.sb + (int64_t)c * Q * sd.sl + h * sd.sh;
  const T* Bg = Bm + b * sB.sb + (int64_t)c * Q * sB.sl + g * sB.sh;
  const TS* sg = dstates + (((b * C + c) * nh + h) * (int64_t)P) * N;
  const float* cbg = cb + (((b * C + c) * ngroups + g) * (int64_t)Q) * Q;

  const int mi = wave & 1, pi0 = wave >> 1;
  floatx16 acc[BPW];
#pragma unroll
  for (int i = 0; i < BPW; ++i) zero_acc(acc[i]);

  // ---- phase A: B . dstates, scaled by the decay to the end of the chunk
  stage_rows<T, 64, N>(Bs, Bg, sB.sl, m0, limit, tid, NoScale());
  {
    constexpr int VPR = N / 4;
#pragma unroll
    for (int i = 0; i < P * VPR / 256; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / VPR, cv = (idx % VPR) * 4;
      const float4 v = state_load4<false>(sg + (int64_t)r * N + cv);
      T* d = Ps + r * S::PC + cv;
      d[0] = (T)v.x, d[1] = (T)v.y, d[2] = (T)v.z, d[3] = (T)v.w;
    }
  }
  if (tid < 64) {
    const ChunkSeq sq = chunk_seq(seq, b, c, Q);
    const bool live = !sq.on() || sq.at(min(m0 + tid, limit - 1)) == sq.at(limit - 1);
    sm[tid] = (m0 + tid < Q && live) ? __expf(fminf(dAp[Q - 1] - dAp[m0 + tid], 0.f)) : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int kk = 0; kk < N; kk += KG) {
    const Vec16<T> a = frag_rows(Bs, S::PC, 32 * mi, kk, lane);
#pragma unroll
    for (int i = 0; i < BPW; ++i) mma_group(a, frag_rows(Ps, S::PC, 32 * (pi0 + 2 * i), kk, lane), acc[i]);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float sc = sm[32 * mi + acc_row(v, lane)];
#pragma unroll
    for (int i = 0; i < BPW; ++i) acc[i][v] *= sc;
  }
  __syncthreads();

  // ---- phase B: the k tiles from the diagonal one to the end of the chunk
  const int ktiles = (limit + 63) / 64;
  for (int kt = mt; kt < ktiles; ++kt) {
    const int k0 = 64 * kt;
    stage_rows<T, 64, P>(Ds, dg, sd.sl, k0, limit, tid, NoScale());
#pragma unroll
    for (int i = 0; i < 64 * 16 / 256; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx >> 4, cv = (idx & 15) * 4;  // row k0 + r of cb, columns m0 + cv ..
      const int k = k0 + r;
      T* d = Wt + r * S::PW + cv;
      // unconditional loads from indices clamped into the chunk
      const bool in = k < limit && m0 + cv < Q;
      const int kc = min(k, limit - 1), mc = min(m0 + cv, Q - 4);
      const float4 w4 = *reinterpret_cast<const float4*>(cbg + (int64_t)kc * Q + mc);
      const float4 a4 = *reinterpret_cast<const float4*>(dAp + mc);
      const float ak = dAp[kc];
      const float w[4] = {w4.x, w4.y, w4.z, w4.w}, am[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        d[e] = (T)((in && k >= m0 + cv + e) ? w[e] * __expf(fminf(ak - am[e], 0.f)) : 0.f);
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 64; kk += KG) {
      const Vec16<T> a = frag_cols(Wt, S::PW, kk, 32 * mi, lane);
#pragma unroll
      for (int i = 0; i < BPW; ++i) mma_group(a, frag_cols(Ds, S::PX, kk, 32 * (pi0 + 2 * i), lane), acc[i]);
    }
    __syncthreads();
  }

  // ---- phase C: through LDS; dx = acc * dt + D * dout, ddt = <acc, x> per row
#pragma unroll
  for (int i = 0; i < BPW; ++i) {
    const int col = 32 * (pi0 + 2 * i) + (lane & 31);
#pragma unroll
    for (int v = 0; v < 16; ++v) Os[(32 * mi + acc_row(v, lane)) * S::PO + col] = acc[i][v];
  }
  __syncthreads();
  constexpr int VPR = P / EPL;
  float dsum[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) dsum[e] = 0.f;
#pragma unroll
  for (int i = 0; i < 64 * VPR / 256; ++i) {
    const int idx = tid + 256 * i;
    const int r = idx / VPR, cv = (idx % VPR) * EPL;
    const int m = m0 + r;
    float dot = 0.f;
    if (m < limit) {
      const int64_t pos = (int64_t)c * Q + m;
      const Vec16<T> xv = load16(x + b * sx.sb + pos * sx.sl + h * sx.sh + cv);
      const float dtm = dtp[m];
      float v[EPL];
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        v[e] = Os[r * S::PO + cv + e];
        dot = fmaf(v[e], xv.get(e), dot);
        v[e] *= dtm;
      }
      if (D) {
        const Vec16<T> dv = load16(dout + b * sd.sb + pos * sd.sl + h * sd.sh + cv);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          v[e] = fmaf(d_has_hdim ? D[h * P + cv + e] : D[h], dv.get(e), v[e]);
          dsum[e] = fmaf(dv.get(e), xv.get(e), dsum[e]);
        }
      }
      Vec16<T> o;
      o.set_all(v);
      store16(dx + b * sdx.sb + pos * sdx.sl + h * sdx.sh + cv, o);
    }
    // the VPR lanes of a row are adjacent: butterfly sum, then one of them writes
#pragma unroll
    for (int off = 1; off < VPR; off <<= 1) dot += __shfl_xor(dot, off);
    if ((idx % VPR) == 0 && m < Q) ddtp[m] = dot;
  }
  if (dslot) store_dD_partial<EPL, VPR>(dslot, dsum, lane);
}

// ------------------------------------------------------------------------------------
// Gradient of the causal term of the chunk scan with respect to the per-position dA, for chunk
// sizes of 64, 128 or 256.  One workgroup per (b, c, h).  With
//   W[m][n] = <dout[m], x[n]> * dt_n * cb[m][n] * exp(min(dA_m - dA_n, 0))   for n < m < limit,
// ddA[j] = sum_{i < j} (colsum_i - rowsum_i).  Wave w owns the 32-row blocks w and MB-1-w (which
// balances the triangle) and walks their column blocks up to the diagonal: <dout, x> on the MFMA
// (dout rows straight from global memory, the chunk's x rows shared through LDS), the weights in
// the accumulator layout, row sums kept per lane, column sums combined through LDS.  The prefix
// sum over the chunk closes the kernel, so nothing else is launched and no workspace is needed.
// ------------------------------------------------------------------------------------
template <typename T, int P>
struct DdaSmem {
  static constexpr int PX = Tile<T>::pitch(P);
  static constexpr int kBytes = 256 * PX * (int)sizeof(T) + (4 * 256 + 256 + 256 + 256) * (int)sizeof(float);
};

template <typename T, int P>
__global__ __launch_bounds__(256) void ssd_ddA_causal_kernel(
    const T* __restrict__ x, Strides3 sx, const T* __restrict__ dout, Strides3 sd, const float* __restrict__ dt,
    const float* __restrict__ dA_cs, const float* __restrict__ cb, float* __restrict__ ddA, int nh,
    int heads_per_group, int ngroups, int L, int Q, int C) {
  using S = DdaSmem<T, P>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, KS = P / KG;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Xs = reinterpret_cast<T*>(smem);
  float* colpart = reinterpret_cast<float*>(smem + 256 * S::PX * sizeof(T));  // [4 waves][256]
  float* rowsum = colpart + 4 * 256;
  float* dAs = rowsum + 256;
  float* dts = dAs + 256;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int h = bid % nh;
  const int c = (bid / nh) % C;
  const int64_t b = bid / ((int64_t)nh * C);
  const int limit = min(Q, L - c * Q);
  const int MB = Q / 32;
  const int64_t chunk = (b * nh + h) * C + c;
  const float* cbg = cb + (((b * C + c) * ngroups + h / heads_per_group) * (int64_t)Q) * Q;
  const T* xg = x + b * sx.sb + (int64_t)c * Q * sx.sl + h * sx.sh;
  const T* dg = dout + b * sd.sb + (int64_t)c * Q * sd.sl + h * sd.sh;

  // (raw buffer of 32-bit words, no bounds to speak of: the offsets stay inside the chunk's Q x Q block)
  const __amdgpu_buffer_rsrc_t cb_desc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(cbg), 0, 0x7fffffff, 0x00020000);

  SSD_TSTAMP(0);
  // shared: the chunk's x rows (zero past the limit), dA, dt; cleared: the sums
  static_assert(S::PX == Tile<T>::pitch(P), "stage_rows writes rows at this pitch");
  if (Q == 256) stage_rows<T, 256, P, NoScale, true>(Xs, xg, sx.sl, 0, limit, tid, NoScale());
  else if (Q == 128) stage_rows<T, 128, P, NoScale, true>(Xs, xg, sx.sl, 0, limit, tid, NoScale());
  else stage_rows<T, 64, P, NoScale, true>(Xs, xg, sx.sl, 0, limit, tid, NoScale());
  if (tid < Q) {
    dAs[tid] = dA_cs[chunk * Q + tid];
    dts[tid] = dt[chunk * Q + tid];
  }
  rowsum[tid] = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) colpart[w * 256 + tid] = 0.f;
  __syncthreads();
  SSD_TSTAMP(1);
  // (a ragged chunk keeps the direct form, whose masks keep whatever cb holds past the sequence out of the sums)
  const bool falling = __syncthreads_and(tid + 1 >= Q || dAs[tid + 1] <= dAs[tid]) != 0 && limit == Q;

#pragma unroll
  for (int slot = 0; slot < 2; ++slot) {
    const int mb = slot == 0 ? wave : MB - 1 - wave;
    if (slot == 1) SSD_TSTAMP(2);
    if (2 * wave >= MB) continue;  // fewer than 8 row blocks: the upper waves have none
    const int m_lane = 32 * mb + l32;  // row whose dout this lane feeds into the MFMA
    Vec16<T> a[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      a[ks] = load16(dg + (int64_t)min(m_lane, limit - 1) * sd.sl + KG * ks + EPL * half);
      if (m_lane >= limit) a[ks].zero();
    }
    // Below the diagonal blocks the decay factors as exp(dA_m - r) * exp(r - dA_n) with r = dA of the
    // block row's first position: where dA does not increase along the chunk (`falling`; it is a cumsum
    // of dt * A with A < 0) both exponents are <= 0 there, so neither factor overflows and the clamp of
    // the exponent at 0 never acts.  That takes the exponential out of the element loop (one per row and
    // block row, one per column and block); the diagonal blocks and any other dA keep the direct form.
    const float r = dAs[32 * mb];
    // the same inside the diagonal block if dA falls by so little over its 32 positions that neither
    // factor leaves the range of float32
    const bool narrow = r - dAs[32 * mb + 31] <= 60.f;
    float rowacc[16], em[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      rowacc[v] = 0.f;
      em[v] = __expf(dAs[32 * mb + acc_row(v, lane)] - r);
    }
    // cb through a buffer descriptor: the part of the address that depends on the accumulator register,
    // the block row and the turn is a scalar offset, the lane's part one register for all sixteen loads
    const int cb_lane = (4 * half * Q + l32) * (int)sizeof(float);
    for (int nb = 0; nb <= mb; ++nb) {
      const int n = 32 * nb + l32;
      // every load is issued before the first use: none of them sits inside a branch
      float cbv[16];
#pragma unroll
      for (int v = 0; v < 16; ++v)
        cbv[v] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
            cb_desc, cb_lane, ((32 * mb + 8 * (v >> 2) + (v & 3)) * Q + 32 * nb) * (int)sizeof(float), 0));
      floatx16 acc;
      zero_acc(acc);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) mma_group(a[ks], frag_rows(Xs, S::PX, 32 * nb, KG * ks, lane), acc);
      const float dAn = dAs[n], wn = dts[n];
      float col = 0.f;
      if (falling && nb < mb) {
        const float gn = wn * __expf(r - dAn);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float u = acc[v] * cbv[v] * em[v];
          rowacc[v] = fmaf(u, gn, rowacc[v]);
          col += u;
        }
        col *= gn;
      } else if (falling && narrow) {  // the diagonal block: exp(r - dA_n) >= 1 here, and bounded
        const float gn = wn * __expf(r - dAn);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float u = n < 32 * mb + acc_row(v, lane) ? acc[v] * cbv[v] * em[v] : 0.f;
          rowacc[v] = fmaf(u, gn, rowacc[v]);
          col += u;
        }
        col *= gn;
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = 32 * mb + acc_row(v, lane);
          const float f = acc[v] * cbv[v] * wn * __expf(fminf(dAs[m] - dAn, 0.f));
          const float w = (n < m && m < limit) ? f : 0.f;
          rowacc[v] += w;
          col += w;
        }
      }
      col += __shfl_xor(col, 32);  // the two halves of the wave hold different rows of one column
      if (half == 0) colpart[wave * 256 + n] += col;
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float t = half_wave_sum(rowacc[v]);
      if (l32 == 31) rowsum[32 * mb + acc_row(v, lane)] = t;
    }
  }
  SSD_TSTAMP(3);
  __syncthreads();
  SSD_TSTAMP(4);
  // delta_i = colsum_i - rowsum_i; ddA[j] = sum_{i<j} delta_i: wave 0, four positions per lane
  if (wave == 0) {
    const int per = (Q + 63) >> 6;
    float d[4], local = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = lane * per + i;
      d[i] = 0.f;
      if (i < per && q < Q)
        d[i] = colpart[q] + colpart[256 + q] + colpart[512 + q] + colpart[768 + q] - rowsum[q];
      local += d[i];
    }
    float run = wave_inclusive_scan(local) - local;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = lane * per + i;
      if (i < per && q < Q) {
        ddA[chunk * Q + q] = run;
        run += d[i];
      }
    }
  }
  SSD_TSTAMP(5);
}

// ------------------------------------------------------------------------------------
// dx / ddt for chunk sizes that are multiples of 256: the mirror image of
// ssd_chunk_scan_wide_kernel.  One workgroup per (b, c, h, 256-row super-tile); wave w owns the
// 32-row blocks w and 7 - w.  The k super-tiles run from the diagonal one to the end of the
// chunk; the weight fragment of a lane (row m, consecutive k) is a column piece of cb, read as
// one 4-byte load per k that is contiguous across the 32 lanes of a half-wave.
// ------------------------------------------------------------------------------------
template <typename T, int P, int N, typename TS>
__global__ __launch_bounds__(256, (P == 64 ? 3 : 2)) void ssd_chunk_scan_bwd_dx_wide_kernel(
    const float* __restrict__ cb, const T* __restrict__ x, Strides3 sx, const T* __restrict__ dout, Strides3 sd,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, const T* __restrict__ Bm, Strides3 sB,
    const TS* __restrict__ dstates, const float* __restrict__ D, int d_has_hdim, T* __restrict__ dx,
    Strides3 sdx, float* __restrict__ ddt, int nh, int heads_per_group, int ngroups, int L, int Q, int C,
    int stiles, SeqIdx seq, float* __restrict__ dD_part) {
  using S = WideSmem<T, P, N>;
  constexpr int EPL = Vec16<T>::N, KG = Tile<T>::KG, PB = P / 32, ST = S::ST;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* Ds = reinterpret_cast<T*>(smem);
  T* Pv = reinterpret_cast<T*>(smem);
  float* Os = reinterpret_cast<float*>(smem);
  float* dAk = reinterpret_cast<float*>(smem + S::kMain);
  float* fk = dAk + ST;  // per-position factor of the weights past the diagonal
  float* sm = dAk + 2 * ST;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, half = lane >> 5;
  const int bid = xcd_local_index((int)blockIdx.x, (int)gridDim.x);
  const int st = bid % stiles;
  const int h = (bid / stiles) % nh;
  const int c = (bid / (stiles * nh)) % C;
  const int64_t b = bid / ((int64_t)stiles * nh * C);
  const int limit = min(Q, L - c * Q);
  const int m0 = ST * st;
  const int64_t chunk = (b * nh + h) * C + c;
  float* ddtp = ddt + chunk * Q;
  // slot of this wave in dD_part (batch, C, nheads, 4 * stiles, hdim)
  float* dslot = dD_part ? dD_part + ((((b * C + c) * nh + h) * (int64_t)stiles + st) * 4 + wave) * P : nullptr;
  if (m0 >= limit) {
    ddtp[m0 + tid] = 0.f;
    if (dslot && lane < P / EPL) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) dslot[lane * EPL + e] = 0.f;
    }
    return;
  }
  const int g = h / heads_per_group;
  const float* dAp = dA_cs + chunk * Q;
  const float* dtp = dt + chunk * Q;
  const T* dg = dout + b * sd.sb + (int64_t)c * Q * sd.sl + h * sd.sh;
  const T* Bg = Bm + b * sB.sb + (int64_t)c * Q * sB.sl + g * sB.sh;
  const TS* sg = dstates + (((b * C + c) * nh + h) * (int64_t)P) * N;
  const float* cbg = cb + (((b * C + c) * ngroups + g) * (int64_t)Q) * Q;

  int mrow[2];
  mrow[0] = 32 * wave;
  mrow[1] = 32 * (7 - wave);
  floatx16 acc[2][PB];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) zero_acc(acc[mb][pb]);

  SSD_TSTAMP(0);
  // ---- phase A: B . dstates, scaled by the decay to the end of the chunk
  {
    constexpr int VPR = N / 4;
#pragma unroll
    for (int i = 0; i < P * VPR / 256; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / VPR, cv = (idx % VPR) * 4;
      const float4 v = state_load4<true>(sg + (int64_t)r * N + cv);
      T* d = Pv + r * S::PC + cv;
      d[0] = (T)v.x, d[1] = (T)v.y, d[2] = (T)v.z, d[3] = (T)v.w;
    }
  }
  {
    const ChunkSeq sq = chunk_seq(seq, b, c, Q);
    const bool live = !sq.on() || sq.at(min(m0 + tid, limit - 1)) == sq.at(limit - 1);
    sm[tid] = live ? __expf(fminf(dAp[Q - 1] - dAp[m0 + tid], 0.f)) : 0.f;
  }
  __syncthreads();
  SSD_TSTAMP(1);
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int m = m0 + mrow[mb] + l32;
    const T* brow = Bg + (int64_t)min(m, limit - 1) * sB.sl + EPL * half;
#pragma unroll
    for (int kk = 0; kk < N; kk += KG) {
      Vec16<T> a = load16(brow + kk);
      if (m >= limit) a.zero();
#pragma unroll
      for (int pb = 0; pb < PB; ++pb) mma_group(a, frag_rows(Pv, S::PC, 32 * pb, kk, lane), acc[mb][pb]);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float sc = sm[mrow[mb] + acc_row(v, lane)];
#pragma unroll
      for (int pb = 0; pb < PB; ++pb) acc[mb][pb][v] *= sc;
    }
  }

  // ---- phase B: the k super-tiles from the diagonal one to the end of the chunk
  SSD_TSTAMP(2);
  __syncthreads();  // the dout tile takes the place of dstates
  SSD_TSTAMP(3);
  for (int kt = st; kt < stiles && ST * kt < limit; ++kt) {
    const int k0 = ST * kt;
    stage_rows<T, ST, P>(Ds, dg, sd.sl, k0, limit, tid, NoScale());
    {
      // Past the diagonal the weight of (m, k) is split at the first position r of k's group of
      // 32: exp(dA_k - dA_r) is one exponential per position k, shared by all rows, and
      // exp(dA_r - dA_m) one per row and group.  Each exponent is clamped at 0 like the whole is
      // in the reference; for a dA_cumsum that is monotone inside the chunk the product is the
      // reference's clamped exponential.  Positions past the end of the sequence get factor 0.
      const float ak = dAp[k0 + tid], ar = dAp[k0 + (tid & ~31)];
      dAk[tid] = ak;
      fk[tid] = k0 + tid < limit ? __expf(fminf(ak - ar, 0.f)) : 0.f;
    }
    __syncthreads();
    SSD_TSTAMP(4);
    const bool diag = kt == st;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int mloc = mrow[mb] + l32;
      const float am = dAp[m0 + mloc];
      const float* cbcol = cbg + (int64_t)k0 * Q + m0 + mloc;  // cb[k0 + k][m]: stride Q along k
      // NS steps at a time (the step count is even): their cb pieces are all requested before the
      // first is used, so the wave waits for memory once per NS steps.  Only where the registers
      // allow it.
      constexpr int NS = (P == 64 && sizeof(T) == 2) ? 2 : 1;
      for (int kk0 = diag ? mrow[mb] : 0; kk0 < ST; kk0 += NS * KG) {
        float w[NS][EPL];
#pragma unroll
        for (int u = 0; u < NS; ++u)
#pragma unroll
          for (int e = 0; e < EPL; ++e) w[u][e] = cbcol[(int64_t)(kk0 + KG * u + EPL * half + e) * Q];
        // the group of 32 positions that holds the diagonal takes the exact, masked form
        const int grp_first = kk0 & ~31;
        const bool exact = diag && grp_first <= mrow[mb] + 31;
        const float gm = __expf(fminf(dAk[grp_first] - am, 0.f));
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const int kk = kk0 + KG * u, kb = kk + EPL * half;
          Vec16<T> a;
          float wf[EPL];
          if (exact) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
              const int k = kb + e;
              const float f = w[u][e] * __expf(fminf(dAk[k] - am, 0.f));
              wf[e] = (k < mloc || k0 + k >= limit) ? 0.f : f;
            }
          } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) wf[e] = w[u][e] * fk[kb + e] * gm;
          }
          a.set_all(wf);
#pragma unroll
          for (int pb = 0; pb < PB; ++pb) mma_group(a, frag_cols(Ds, S::PX, kk, 32 * pb, lane), acc[mb][pb]);
        }
      }
    }
    SSD_TSTAMP(5);
    __syncthreads();
  }
  SSD_TSTAMP(6);

  // ---- phase C: each wave moves its two blocks through its own staging area.  The rows of x
  // (and dout, dt) that the block's results meet are requested before the accumulators go to
  // LDS, so that their latency hides behind the staging (where that takes at most four pieces
  // per lane; otherwise they are fetched as they are needed).
  float* mine = Os + wave * 32 * S::PO;
  constexpr int VPR = P / EPL, NI = 32 * VPR / 64;
  constexpr bool kEarly = NI <= 4;
  float dsum[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) dsum[e] = 0.f;
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    Vec16<T> xv[kEarly ? NI : 1], dv[kEarly ? NI : 1];
    float dtm[kEarly ? NI : 1];
    if constexpr (kEarly) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int idx = lane + 64 * i;
        const int r = idx / VPR, cv = (idx % VPR) * EPL;
        const int m = m0 + mrow[mb] + r;
        const int64_t pos = (int64_t)c * Q + min(m, limit - 1);
        xv[i] = load16_stream(x + b * sx.sb + pos * sx.sl + h * sx.sh + cv);
        dtm[i] = dtp[m];
        if (D) dv[i] = load16(dout + b * sd.sb + pos * sd.sl + h * sd.sh + cv);
      }
    }
#pragma unroll
    for (int pb = 0; pb < PB; ++pb)
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[acc_row(v, lane) * S::PO + 32 * pb + l32] = acc[mb][pb][v];
    __builtin_amdgcn_s_waitcnt(0xc07f);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int idx = lane + 64 * i;
      const int r = idx / VPR, cv = (idx % VPR) * EPL;
      const int m = m0 + mrow[mb] + r;
      const int64_t pos = (int64_t)c * Q + min(m, limit - 1);
      Vec16<T> xi, di;
      float dti;
      if constexpr (kEarly) {
        xi = xv[i], di = dv[i], dti = dtm[i];
      } else {
        xi = load16_stream(x + b * sx.sb + pos * sx.sl + h * sx.sh + cv);
        dti = dtp[m];
        if (D) di = load16(dout + b * sd.sb + pos * sd.sl + h * sd.sh + cv);
      }
      float dot = 0.f, v[EPL];
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        v[e] = mine[r * S::PO + cv + e];
        dot = fmaf(v[e], xi.get(e), dot);
        v[e] *= dti;
      }
      if (m >= limit) dot = 0.f;
      if (D) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          v[e] = fmaf(d_has_hdim ? D[h * P + cv + e] : D[h], di.get(e), v[e]);
          if (m < limit) dsum[e] = fmaf(di.get(e), xi.get(e), dsum[e]);
        }
      }
      if (m < limit) {
        Vec16<T> o;
        o.set_all(v);
        store16_stream(dx + b * sdx.sb + pos * sdx.sl + h * sdx.sh + cv, o);
      }
#pragma unroll
      for (int off = 1; off < VPR; off <<= 1) dot += __shfl_xor(dot, off);
      if ((idx % VPR) == 0) ddtp[m] = dot;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  if (dslot) store_dD_partial<EPL, VPR>(dslot, dsum, lane);
  SSD_TSTAMP(7);
}

// ------------------------------------------------------------------------------------
// States at the end of each sequence of a packed batch: for sequence s ending at position e
// (exclusive) in chunk c = (e - 1) / Q, the positions of s that lie in chunk c weighted by the decay
// to e - 1 and dt, plus the state entering chunk c decayed to e - 1 when s began before that chunk
// (_chunk_state_varlen_kernel, kernels/ema_chunk_state.py:500-575 of the reference).  A handful of
// sequences per call: plain fp32 multiply-adds on 64 x 64 tiles of the state, 4 x 4 per thread.
// Grid (P tiles * N tiles, sequences, heads).  The weighted B is rounded to T before the product,
// as the reference does; an empty or out-of-range sequence gives zeros.
// ------------------------------------------------------------------------------------
template <typename T, typename TS>
__global__ __launch_bounds__(256) void ssd_chunk_state_varlen_kernel(
    const T* __restrict__ x, int64_t x_sl, int64_t x_sh, const T* __restrict__ Bm, int64_t b_sl, int64_t b_sg,
    const float* __restrict__ dt, const float* __restrict__ dA_cs, const TS* __restrict__ chunk_states,
    const int32_t* __restrict__ cu_seqlens, float* __restrict__ out, int L, int nh, int hpg, int P, int N, int Q,
    int C) {
  constexpr int TP = 64, TN = 64, KB = 32;
  __shared__ float sx[KB][TP];
  __shared__ float sb[KB][TN];
  __shared__ float ss[KB];
  const int tid = threadIdx.x;
  const int tiles_n = (N + TN - 1) / TN;
  const int p0 = (blockIdx.x / tiles_n) * TP, n0 = (blockIdx.x % tiles_n) * TN;
  const int s = blockIdx.y, h = blockIdx.z;
  const int tp = (tid >> 4) * 4, tn = (tid & 15) * 4;
  const int start = cu_seqlens[s];
  const int end = min(cu_seqlens[s + 1], L);
  float acc[4][4] = {};
  const bool live = start >= 0 && end > start;  // uniform over the workgroup
  const int c = live ? (end - 1) / Q : 0;
  const int limit = end - c * Q;                // positions of chunk c up to the sequence's end
  const int first = max(start - c * Q, 0);      // first position of chunk c that belongs to s
  const int64_t row = ((int64_t)h * C + c) * Q;  // dt, dA_cumsum are (nheads, nchunks, Q)
  const float dA_last = live ? dA_cs[row + limit - 1] : 0.f;
  const T* xg = x + (int64_t)c * Q * x_sl + (int64_t)h * x_sh;
  const T* bg = Bm + (int64_t)c * Q * b_sl + (int64_t)(h / hpg) * b_sg;
  for (int k0 = live ? (first / KB) * KB : limit; k0 < limit; k0 += KB) {
    if (tid < KB) {
      const int k = k0 + tid;
      const int kc = min(k, limit - 1);
      const float w = __expf(fminf(dA_last - dA_cs[row + kc], 0.f)) * dt[row + kc];
      ss[tid] = (k >= first && k < limit) ? w : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < KB * TP / 256; ++i) {
      const int idx = tid + i * 256;
      const int kk = idx / TP, col = idx % TP;
      const int kc = min(k0 + kk, limit - 1);
      const float w = ss[kk];
      const float xv = (float)xg[(int64_t)kc * x_sl + min(p0 + col, P - 1)];
      const float bv = (float)bg[(int64_t)kc * b_sl + min(n0 + col, N - 1)];
      sx[kk][col] = (w != 0.f && p0 + col < P) ? xv : 0.f;
      sb[kk][col] = (w != 0.f && n0 + col < N) ? (float)(T)(bv * w) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < KB; ++kk) {
      const float4 a = *reinterpret_cast<const float4*>(&sx[kk][tp]);
      const float4 b = *reinterpret_cast<const float4*>(&sb[kk][tn]);
      const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
  const bool carried = live && start < c * Q;  // the sequence began before chunk c
  const float keep = carried ? __expf(dA_last) : 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = p0 + tp + i, n = n0 + tn + j;
      if (p < P && n < N) {
        float v = acc[i][j];
        if (carried) v = fmaf((float)chunk_states[(((int64_t)c * nh + h) * P + p) * N + n], keep, v);
        out[(((int64_t)s * nh + h) * P + p) * N + n] = v;
      }
    }
}

}  // namespace ssd
