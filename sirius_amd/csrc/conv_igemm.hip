// Implicit-GEMM convolution for gfx950: forward, data gradient and weight
// gradient over NHWC activations and KRSC filters, on the 32x32 MFMA tiles
// (v_mfma_f32_32x32x16_bf16 for bf16 storage, v_mfma_f32_32x32x2_f32 for fp32),
// fp32 accumulation, operands staged through LDS in 16-byte chunks.
//
// The reference has no convolution code of its own: its training scripts call
// torchvision's ResNet (train/resnet152.py:22) and the arithmetic is
// F.conv2d / its autograd formulas.  These kernels restate that arithmetic:
//   FWD    y[n,ho,wo,k]  = sum_{r,s,c} x[n, ho*st-p+r, wo*st-p+s, c] * w[k,r,s,c]
//   DGRAD  dx[n,h,w,c]   = sum_{r,s,k} dy[n,(h+p-r)/st,(w+p-s)/st,k] * wt[c,r,s,k]
//   WGRAD  dw[k,r,s,c]   = sum_{n,ho,wo} dy[n,ho,wo,k] * x[n, ho*st-p+r, wo*st-p+s, c]
//
// GEMM view (rows x cols, reduction):
//   FWD    (N*Ho*Wo) x K,        over R*S*C
//   DGRAD  (N*H*W)   x C,        over R*S*K     (filter pre-transposed to [C][R][S][K])
//   WGRAD  K         x (R*S*C),  over N*Ho*Wo, split across workgroups
//
// FWD / DGRAD: a tile row in LDS holds one GEMM row (or column) and BK reduction
// elements = 4 chunks of 16 bytes (+1 chunk of padding); a lane's MFMA operand is
// one chunk (lanes 0-31 chunk 2j, lanes 32-63 chunk 2j+1 of their row).
//
// WGRAD: both operands are contiguous along the GEMM row/column (channels) and
// strided along the reduction (pixels), the opposite of what an MFMA operand
// wants.  The tiles are kept as they come, [pixel][channel], and the operand is
// formed by the LDS transpose read of gfx950 (ds_read_b64_tr_b16): a group of 16
// lanes reads a 4-pixel x 16-channel block and every lane receives the 4 pixels
// of ONE channel.
//
// The MFMA is issued with the filter-side fragment as the first operand, so a
// lane's 16 accumulators belong to ONE output row and to groups of 4 consecutive
// output columns: the epilogue moves them through LDS as 16-byte vectors and
// writes (and reads the residual / mask) as full 16-byte chunks per lane.
#include "kernels.h"
#include <algorithm>
#include <vector>

#include "context.h"
#include "ops.h"

#include <mutex>
#include <string>

namespace tch {
namespace {

constexpr int kLdsStride = 5;  // FWD/DGRAD: chunks per LDS tile row: 4 data + 1 pad
constexpr int kRowPad = 4;     // WGRAD: chunks of padding per [pixel] row (64 bytes)
constexpr int kStagePad = 4;   // epilogue staging: floats of padding per row

enum Mode : int { kFwd = 0, kDgrad = 1, kWgrad = 2 };

struct IgemmArgs {
  const void* a_src;  // FWD: x        DGRAD: dy       WGRAD: dy
  const void* b_src;  // FWD: w        DGRAD: wt       WGRAD: x
  void* out;          // FWD: y        DGRAD: dx       WGRAD: dw (fp32) or split partials
  const void* add;    // optional addend, laid out like out (FWD/DGRAD)
  const void* mask;   // optional: addend counts only where mask > 0
  int add_sub;        // DGRAD: 1 = `add` lives on the stride-2 subsampled pixel grid [N, ceil(H/2), ceil(W/2), C] and
                      // counts at the even (h, w) only (the data gradient of a strided 1x1 convolution, kept compact)
  const float* bias;  // optional per-column bias (FWD)
  const float* scale; // optional per-column factor applied before the bias (FWD: an inference-mode BatchNorm folded in)
  int relu_out;       // FWD: the stored output is max(0, .) of everything above
  float* dbias;       // WGRAD, optional: column sums of dy (the gradient of that bias), [splits][K] partials or final
  float* stats;       // optional: per (row tile, column) pair of sums over the stored output (see finish_tile)
  long long* stat_acc;  // optional, instead of stats: the same pair added to exact accumulators, [copies][4][columns]
  int stat_acc_copies;  // power of two
  const void* bn_mask;      // DGRAD with stats, optional: the stored output is zeroed where bn_mask <= 0
  const void* bn_x;         // DGRAD with stats: input of the BatchNorm this gradient flows into, laid out like out
  const float* bn_mean;     // DGRAD with stats: that BatchNorm's saved batch mean / inverse std per column
  const float* bn_invstd;
  // Optional, with stats: the workgroup that finishes a column tile last also turns the sums into the
  // BatchNorm's per-channel coefficients (no finalize launch).  fin_counters: one int per column tile,
  // zero before the launch; the finishing workgroup leaves it zero again.
  int* fin_counters;
  const float* fin_gamma;
  const float* fin_beta;     // FWD
  float* fin_running_mean;   // FWD, may be null (then fin_running_var is null too)
  float* fin_running_var;
  float* fin_out0;           // FWD: saved batch mean         DGRAD: dgamma
  float* fin_out1;           // FWD: saved inverse std        DGRAD: dbeta
  float* fin_coef;           // FWD: scale[C], shift[C]       DGRAD: coef[3][C] (dx = c0*g + c1*x + c2)
  float fin_momentum, fin_eps;
  int fin_accumulate;        // DGRAD: dgamma / dbeta +=
  int N, H, W, C;     // x side
  int Ho, Wo, K;      // y side
  int R, S, stride, stride_log2, pad;
  int gemm_m, gemm_n, gemm_k;
  int tiles_m, tiles_n, splits;
  int group_rows;   // FWD/DGRAD direct-to-LDS kernel: row tiles per group of the tile order (0 / 1: row-major)
  int k_per_split;  // multiple of BK
  int out_f32;      // FWD/DGRAD: store fp32 instead of T
  int accumulate;   // WGRAD with splits == 1: out += result
  int take_pending; // WGRAD, read by the launcher only: the context's pending split reduction rides this launch
  int pointwise;    // 1x1, stride 1, pad 0
  uint32_t a_bytes, b_bytes;  // extents of a_src / b_src for the bounds-checked buffer loads
  FastDiv div_plane;  // pixels per image on the gather side
  FastDiv div_width;  // row width on the gather side
};

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4_t* lds_short4_ptr;
union TrPart {
  short4_t s;
  uint32_t w[2];
};

// first operand = filter-side fragment (its rows become accumulator registers),
// second operand = activation-side fragment (its rows become accumulator lanes)
template <typename T>
__device__ inline void mma(const Chunk& first, const Chunk& second, f32x16_t& acc);
template <>
__device__ inline void mma<bf16>(const Chunk& first, const Chunk& second, f32x16_t& acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(first.h, second.h, acc, 0, 0, 0);
}
template <>
__device__ inline void mma<float>(const Chunk& first, const Chunk& second, f32x16_t& acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(first.f[e], second.f[e], acc, 0, 0, 0);
}

// Operand loads go through buffer instructions: an offset outside the declared extent
// returns zeros, so padding, ragged edges and the tail of the reduction need neither a
// branch nor a select, and the loads stay in flight across the multiply of earlier tiles.
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
constexpr uint32_t kOutOfRange = 0x80000000u;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

__device__ inline Chunk load_chunk(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off, bool valid) {
  uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(valid ? byte_off : kOutOfRange), 0, 0);
  Chunk c;
  c.w[0] = v[0];
  c.w[1] = v[1];
  c.w[2] = v[2];
  c.w[3] = v[3];
  return c;
}

// Walks the reduction index of a filter-tap-major operand: (r, s, channel) with
// `channels` per tap, advancing by a fixed step; no division after init.
struct TapWalker {
  int r, s, ch;
  __device__ inline void init(int k, int channels, int S) {
    int tap = k / channels;
    ch = k - tap * channels;
    r = tap / S;
    s = tap - r * S;
  }
  // branch-free; a step covers at most 4 taps (channels >= one chunk, step = 4 chunks)
  __device__ inline void advance(int step, int channels, int S) {
    ch += step;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool wrap = ch >= channels;
      ch -= wrap ? channels : 0;
      s += wrap ? 1 : 0;
      const bool wrap_s = s >= S;
      s = wrap_s ? 0 : s;
      r += wrap_s ? 1 : 0;
    }
  }
};

// Called by every workgroup after it has stored its row of partial sums: the one that arrives last at
// the column tile's counter sums all tiles_m rows of its BN columns (fp64, fixed order) and writes
// the BatchNorm coefficients.  Nobody waits for anybody: a workgroup that is not last just leaves.
// Visibility across the chip's L2 slices without flushing them (a device-scope fence per workgroup
// writes back every dirty line of its L2 slice, the convolution's own output included, and costs
// more than the whole kernel): the partial sums are published with device-scope atomic exchanges,
// whose result the publishing thread waits for before the barrier that precedes the counter bump,
// and the finishing workgroup reads them with device-scope atomic loads.  Atomics execute at the
// point all slices share.
template <int MODE, int BN, int NT>
__device__ inline void finalize_column_tile(const IgemmArgs& p, float* stage, int tid, int n0) {
  __shared__ int last_arrival;
  __syncthreads();
  if (tid == 0) {
    int* counter = p.fin_counters + n0 / BN;
    const int prev = atomicAdd(counter, 1);
    last_arrival = prev == p.tiles_m - 1;
    if (last_arrival) *counter = 0;  // every other workgroup of this column tile has been here already
  }
  __syncthreads();
  if (!last_arrival) return;

  constexpr int PARTS = NT / BN;   // row tiles are dealt round-robin to PARTS threads per column
  const int cl = tid % BN, part = tid / BN;
  double s_part = 0.0, q_part = 0.0;
  if (n0 + cl < p.gemm_n) {
    constexpr int U = 8;
    for (int b = part; b < p.tiles_m; b += U * PARTS) {
      unsigned long long v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int bb = b + u * PARTS;
        v[u] = bb < p.tiles_m
                   ? __hip_atomic_load(reinterpret_cast<const unsigned long long*>(
                                           p.stats + (static_cast<int64_t>(bb) * p.gemm_n + n0 + cl) * 2),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                   : 0ull;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        s_part += __uint_as_float(static_cast<uint32_t>(v[u]));
        q_part += __uint_as_float(static_cast<uint32_t>(v[u] >> 32));
      }
    }
  }
  double* red = reinterpret_cast<double*>(stage);  // [PARTS][BN][2]
  red[(part * BN + cl) * 2] = s_part;
  red[(part * BN + cl) * 2 + 1] = q_part;
  __syncthreads();
  const int c = n0 + tid;
  if (tid >= BN || c >= p.gemm_n) return;
  double s = 0.0, q = 0.0;
#pragma unroll
  for (int k = 0; k < PARTS; ++k) {
    s += red[(k * BN + tid) * 2];
    q += red[(k * BN + tid) * 2 + 1];
  }
  const double n = static_cast<double>(p.gemm_m);
  const int C = p.gemm_n;
  if (MODE == kFwd) {
    // s = sum x, q = sum x^2  (torch.nn.BatchNorm2d in training mode: biased variance normalises,
    // the unbiased one goes into running_var)
    const double mean = s / n;
    double var = q / n - mean * mean;
    if (var < 0.0) var = 0.0;
    const float invstd = 1.0f / sqrtf(static_cast<float>(var) + p.fin_eps);
    p.fin_out0[c] = static_cast<float>(mean);
    p.fin_out1[c] = invstd;
    if (p.fin_running_mean) {
      const double unbiased = p.gemm_m > 1 ? var * n / (n - 1.0) : var;
      p.fin_running_mean[c] = (1.f - p.fin_momentum) * p.fin_running_mean[c] + p.fin_momentum * static_cast<float>(mean);
      p.fin_running_var[c] = (1.f - p.fin_momentum) * p.fin_running_var[c] + p.fin_momentum * static_cast<float>(unbiased);
    }
    const float sc = p.fin_gamma[c] * invstd;
    p.fin_coef[c] = sc;
    p.fin_coef[C + c] = p.fin_beta[c] - static_cast<float>(mean) * sc;
  } else {
    // s = sum g, q = sum g * xhat
    const float db = static_cast<float>(s), dg = static_cast<float>(q);
    p.fin_out1[c] = p.fin_accumulate ? p.fin_out1[c] + db : db;
    p.fin_out0[c] = p.fin_accumulate ? p.fin_out0[c] + dg : dg;
    const double invstd = p.bn_invstd[c];
    const double scale = static_cast<double>(p.fin_gamma[c]) * invstd;
    const double cb = -scale * invstd * (q / n);
    const double c0 = -scale * (s / n) - cb * p.bn_mean[c];
    p.fin_coef[c] = static_cast<float>(scale);
    p.fin_coef[C + c] = static_cast<float>(cb);
    p.fin_coef[2 * C + c] = static_cast<float>(c0);
  }
}

// The accumulators of one workgroup tile, one 32-row band (index tm) at a time:
// lanes write float4 groups into the staging tile [WM*32][BN + pad], then every
// thread takes E consecutive columns of one row and hands them to `fin` together with the
// number of the visit (tm * ITERS + it, a compile-time constant after unrolling).
template <typename T, int WM, int WN, int TM, int TN, typename Fin>
__device__ inline void staged_epilogue(f32x16_t (&acc)[TM][TN], float* stage, int tid, Fin fin) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int BN = WN * TN * 32;
  constexpr int NT = WM * WN * 64;
  constexpr int LD = BN + kStagePad;
  constexpr int CH = BN / E;
  constexpr int ITERS = (WM * 32 * CH) / NT;
  static_assert((WM * 32 * CH) % NT == 0, "epilogue mapping");
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    __syncthreads();
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int r = wm * 32 + (lane & 31);
        const int c = (wn * TN + tn) * 32 + 8 * j + 4 * (lane >> 5);
        float4 v = make_float4(acc[tm][tn][4 * j], acc[tm][tn][4 * j + 1], acc[tm][tn][4 * j + 2],
                               acc[tm][tn][4 * j + 3]);
        *reinterpret_cast<float4*>(stage + r * LD + c) = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int q = tid + it * NT;
      const int r = q / CH, cc = q - r * CH;
      float v[E];
#pragma unroll
      for (int e = 0; e < E; e += 4) {
        float4 t = *reinterpret_cast<const float4*>(stage + r * LD + cc * E + e);
        v[e] = t.x;
        v[e + 1] = t.y;
        v[e + 2] = t.z;
        v[e + 3] = t.w;
      }
      fin(tm * ITERS + it, ((r >> 5) * TM + tm) * 32 + (r & 31), cc * E, v);
    }
  }
}

template <int E>
__device__ inline void store_floats(float* dst, const float* v) {
#pragma unroll
  for (int e = 0; e < E; e += 4) *reinterpret_cast<float4*>(dst + e) = make_float4(v[e], v[e + 1], v[e + 2], v[e + 3]);
}

// ---------------------------------------------------------------------------
// epilogue of forward / data gradient: bias, gated residual, rounding, 16-byte accesses per
// lane; optionally the sums a BatchNorm next to the convolution needs, one pair per (row tile,
// column) at stats[(tile_m * gemm_n + col) * 2], summed in a fixed order:
//   forward:       sum and sum of squares of the values AS STORED (after rounding to T): the
//                  batch statistics of the BatchNorm that follows;
//   data gradient: the output g is the gradient behind a BatchNorm(+ReLU): it is rounded to T,
//                  zeroed where bn_mask <= 0 (the ReLU), stored, and the pair is sum(g) and
//                  sum(g * xhat), xhat = (bn_x - mean) * invstd: the two reductions of the
//                  BatchNorm backward.
// ---------------------------------------------------------------------------
template <typename T, int MODE, int WM, int WN, int TM, int TN>
__device__ inline void finish_tile(const IgemmArgs& p, f32x16_t (&acc)[TM][TN], float* stage, int tid, int m0, int n0,
                                   int tile_m) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int BN = WN * TN * 32;
  constexpr int NT = WM * WN * 64;
  constexpr int CH = BN / E;   // column chunks of the tile; a thread always gets chunk tid % CH
  constexpr int ROWS = NT / CH;
  static_assert(NT % CH == 0, "stats mapping");
  const bool want_stats = p.stats != nullptr || p.stat_acc != nullptr;
  float st_sum[E], st_sq[E];
#pragma unroll
  for (int e = 0; e < E; ++e) st_sum[e] = st_sq[e] = 0.f;
  // data gradient with BatchNorm sums: the chunks of bn_x and bn_mask this thread will meet are
  // requested up front, so that their latency overlaps the staging of the accumulators
  constexpr int ITERS = (WM * 32 * CH) / NT;
  constexpr int VISITS = TM * ITERS;
  float bn_mu[E], bn_is[E];
  uint4 pre_x[VISITS], pre_m[VISITS];
  if (MODE == kDgrad && want_stats) {
    const int col = n0 + (tid % CH) * E;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      bn_mu[e] = col < p.gemm_n ? p.bn_mean[col + e] : 0.f;
      bn_is[e] = col < p.gemm_n ? p.bn_invstd[col + e] : 0.f;
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int q = tid + it * NT;
        const int r = q / CH;
        const int row = m0 + ((r >> 5) * TM + tm) * 32 + (r & 31);
        const bool ok = row < p.gemm_m && col < p.gemm_n;
        const int64_t idx = static_cast<int64_t>(row) * p.gemm_n + col;
        pre_x[tm * ITERS + it] = ok ? *reinterpret_cast<const uint4*>(static_cast<const T*>(p.bn_x) + idx) : make_uint4(0, 0, 0, 0);
        pre_m[tm * ITERS + it] = (ok && p.bn_mask) ? *reinterpret_cast<const uint4*>(static_cast<const T*>(p.bn_mask) + idx)
                                                   : make_uint4(0, 0, 0, 0);
      }
  }

  staged_epilogue<T, WM, WN, TM, TN>(acc, stage, tid, [&](int visit, int tr, int tc, float* v) {
    const int row = m0 + tr, col = n0 + tc;
    if (row >= p.gemm_m || col >= p.gemm_n) return;
    const int64_t idx = static_cast<int64_t>(row) * p.gemm_n + col;
    if (MODE == kFwd && p.scale) {
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] *= p.scale[col + e];
    }
    if (MODE == kFwd && p.bias) {
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] += p.bias[col + e];
    }
    bool add_here = p.add != nullptr;
    int64_t add_idx = idx;
    if (MODE == kDgrad && p.add_sub && add_here) {
      uint32_t img, rem, h, w;
      p.div_plane.divmod(static_cast<uint32_t>(row), img, rem);
      p.div_width.divmod(rem, h, w);
      add_here = ((h | w) & 1u) == 0u;
      const int64_t hs = (p.H + 1) >> 1, ws = (p.W + 1) >> 1;
      add_idx = ((static_cast<int64_t>(img) * hs + (h >> 1)) * ws + (w >> 1)) * p.gemm_n + col;
    }
    if (add_here) {
      Chunk ca;
      ca.u = *reinterpret_cast<const uint4*>(static_cast<const T*>(p.add) + add_idx);
      float a[E];
      chunk_to_float<T>(ca, a);
      if (p.mask) {
        Chunk cm;
        cm.u = *reinterpret_cast<const uint4*>(static_cast<const T*>(p.mask) + idx);
        float m[E];
        chunk_to_float<T>(cm, m);
#pragma unroll
        for (int e = 0; e < E; ++e)
          if (!(m[e] > 0.f)) a[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] += a[e];
    }
    if (MODE == kFwd && p.relu_out) {
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] = fmaxf(v[e], 0.f);
    }
    if (p.out_f32) {
      store_floats<E>(static_cast<float*>(p.out) + idx, v);
    } else if (MODE == kDgrad && want_stats) {
      Chunk c = float_to_chunk<T>(v);
      chunk_to_float<T>(c, v);
      Chunk cx;
      cx.u = pre_x[visit];
      if (p.bn_mask) {
        Chunk cm;
        cm.u = pre_m[visit];
        float m[E];
        chunk_to_float<T>(cm, m);
#pragma unroll
        for (int e = 0; e < E; ++e)
          if (!(m[e] > 0.f)) v[e] = 0.f;
        c = float_to_chunk<T>(v);  // exact: every v[e] is a value of T
      }
      *reinterpret_cast<uint4*>(static_cast<T*>(p.out) + idx) = c.u;
      float x[E];
      chunk_to_float<T>(cx, x);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        st_sum[e] += v[e];
        st_sq[e] += v[e] * ((x[e] - bn_mu[e]) * bn_is[e]);
      }
    } else {
      const Chunk c = float_to_chunk<T>(v);
      *reinterpret_cast<uint4*>(static_cast<T*>(p.out) + idx) = c.u;
      if (want_stats) {
        chunk_to_float<T>(c, v);  // the statistics are those of the stored values
#pragma unroll
        for (int e = 0; e < E; ++e) {
          st_sum[e] += v[e];
          st_sq[e] += v[e] * v[e];
        }
      }
    }
  });

  if (want_stats) {
    // threads tid, tid + CH, tid + 2 CH, ... hold partial sums of the same E columns
    __syncthreads();
    // [2][E] planes of one float per thread, plane stride NT + 8 floats: the 64 lanes of a store hit 64 consecutive
    // banks, and the 64 lanes of a load below (8 values of e x 8 values of cc) land 8 banks apart per plane: neither
    // has a bank conflict (a [thread][2E] layout made every store a 16-way one)
    constexpr int PS = NT + 8;
    static_assert(2 * E * PS * 4 <= WM * 32 * (BN + kStagePad) * 4, "the sums fit the staging tile");
    float* red = stage;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      red[e * PS + tid] = st_sum[e];
      red[(E + e) * PS + tid] = st_sq[e];
    }
    __syncthreads();
    if (tid < BN) {
      const int cc = tid / E, e = tid - cc * E;
      float a = 0.f, b = 0.f;
#pragma unroll 4
      for (int r = 0; r < ROWS; ++r) {   // thread r * CH + cc holds row group r of chunk column cc
        a += red[e * PS + r * CH + cc];
        b += red[(E + e) * PS + r * CH + cc];
      }
      const int col = n0 + tid;
      if (col < p.gemm_n && p.stat_acc) {
        // every row tile adds to the same pair of accumulators: no per-tile partials, nothing to sum up later
        acc_add2(p.stat_acc, p.gemm_n, p.stat_acc_copies, tile_m, col, a, b);
      } else if (col < p.gemm_n) {
        float2* dst = reinterpret_cast<float2*>(p.stats + (static_cast<int64_t>(tile_m) * p.gemm_n + col) * 2);
        if (p.fin_counters) {
          // published for the workgroup that finishes this column tile (see finalize_column_tile)
          const unsigned long long bits = static_cast<unsigned long long>(__float_as_uint(a)) |
                                          (static_cast<unsigned long long>(__float_as_uint(b)) << 32);
          const unsigned long long old = atomicExch(reinterpret_cast<unsigned long long*>(dst), bits);
          asm volatile("" ::"v"(old));  // wait for the exchange itself, not only for its issue
        } else {
          *dst = make_float2(a, b);
        }
      }
    }
    if (p.fin_counters) finalize_column_tile<MODE, BN, NT>(p, stage, tid, n0);
  }
}

// ---------------------------------------------------------------------------
// forward / data gradient
// ---------------------------------------------------------------------------
template <typename T, int MODE, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM* WN * 64) void igemm_kernel(IgemmArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int BK = 4 * E;
  constexpr int BM = WM * TM * 32;
  constexpr int BN = WN * TN * 32;
  constexpr int NT = WM * WN * 64;
  constexpr int EB = sizeof(T);
  constexpr int A_PT = (BM * 4) / NT;
  constexpr int B_PT = (BN * 4) / NT;
  static_assert((BM * 4) % NT == 0 && (BN * 4) % NT == 0, "tile/loader mismatch");
  constexpr int OPER_BYTES = (BM + BN) * kLdsStride * 16 * 2;
  constexpr int STAGE_BYTES = WM * 32 * (BN + kStagePad) * 4;
  constexpr int LDS_BYTES = OPER_BYTES > STAGE_BYTES ? OPER_BYTES : STAGE_BYTES;

  __shared__ uint4 lds[LDS_BYTES / 16];
  uint4* lds_a = lds;                            // [2][BM * kLdsStride]
  uint4* lds_b = lds + 2 * BM * kLdsStride;      // [2][BN * kLdsStride]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  uint32_t id = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = id / p.tiles_n;
  const int tile_n = id - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int k_end = p.gemm_k;
  const int nk = (k_end + BK - 1) / BK;

  // ---- operand A: gather of activation rows; the chunk column is the same for every i ----
  const int in_h = (MODE == kFwd) ? p.H : p.Ho;
  const int in_w = (MODE == kFwd) ? p.W : p.Wo;
  const int in_c = (MODE == kFwd) ? p.C : p.K;
  const int chunk_col = tid & 3;
  int a_base[A_PT], a_h0[A_PT], a_w0[A_PT];
  bool a_row_ok[A_PT];
  TapWalker walk;
  walk.init(chunk_col * E, in_c, p.S);
#pragma unroll
  for (int i = 0; i < A_PT; ++i) {
    const int row = m0 + ((tid + i * NT) >> 2);
    a_row_ok[i] = row < p.gemm_m;
    uint32_t img = 0, pix = 0, oh = 0, ow = 0;
    if (a_row_ok[i]) {
      p.div_plane.divmod(static_cast<uint32_t>(row), img, pix);
      p.div_width.divmod(pix, oh, ow);
    }
    if (p.pointwise) {
      a_base[i] = row * in_c;  // dense [gemm_m][in_c]
      a_h0[i] = a_w0[i] = 0;
    } else {
      a_base[i] = static_cast<int>(img) * in_h * in_w * in_c;
      if (MODE == kFwd) {
        a_h0[i] = static_cast<int>(oh) * p.stride - p.pad;
        a_w0[i] = static_cast<int>(ow) * p.stride - p.pad;
      } else {
        a_h0[i] = static_cast<int>(oh) + p.pad;
        a_w0[i] = static_cast<int>(ow) + p.pad;
      }
    }
  }

  // two register sets: the tiles kt+1 and kt+2 are in flight while tile kt is multiplied
  Chunk ra0[A_PT], rb0[B_PT], ra1[A_PT], rb1[B_PT];
  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a_src, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b_src, p.b_bytes);

  auto load_tiles = [&](int kt, Chunk* ra, Chunk* rb) {
    const int k0 = kt * BK;
    const int kk = k0 + chunk_col * E;
    if (p.pointwise) {
      const bool k_ok = kk < k_end;
#pragma unroll
      for (int i = 0; i < A_PT; ++i)
        ra[i] = load_chunk(rsrc_a, static_cast<uint32_t>(a_base[i] + kk) * EB, a_row_ok[i] && k_ok);
    } else {
      const bool tap_ok = walk.r < p.R && kk < k_end;
#pragma unroll
      for (int i = 0; i < A_PT; ++i) {
        int hi, wi;
        bool ok = a_row_ok[i] && tap_ok;
        if (MODE == kFwd) {
          hi = a_h0[i] + walk.r;
          wi = a_w0[i] + walk.s;
        } else {
          const int th = a_h0[i] - walk.r, tw = a_w0[i] - walk.s;
          const int sm = p.stride - 1;
          ok = ok && th >= 0 && tw >= 0 && ((th & sm) == 0) && ((tw & sm) == 0);
          hi = th >> p.stride_log2;
          wi = tw >> p.stride_log2;
        }
        ok = ok && static_cast<unsigned>(hi) < static_cast<unsigned>(in_h) &&
             static_cast<unsigned>(wi) < static_cast<unsigned>(in_w);
        const uint32_t off = static_cast<uint32_t>(a_base[i] + (hi * in_w + wi) * in_c + walk.ch) * EB;
        ra[i] = load_chunk(rsrc_a, off, ok);
      }
      walk.advance(BK, in_c, p.S);
    }
    // operand B: dense filter rows: FWD reads w[K][R*S*C], DGRAD reads wt[C][R*S*K]
#pragma unroll
    for (int i = 0; i < B_PT; ++i) {
      const int row = n0 + ((tid + i * NT) >> 2);
      const bool ok = row < p.gemm_n && kk < k_end;
      rb[i] = load_chunk(rsrc_b, static_cast<uint32_t>(row * p.gemm_k + kk) * EB, ok);
    }
  };

  auto store_tiles = [&](int buf, const Chunk* ra, const Chunk* rb) {
#pragma unroll
    for (int i = 0; i < A_PT; ++i) {
      const int q = tid + i * NT;
      lds_a[buf * BM * kLdsStride + (q >> 2) * kLdsStride + (q & 3)] = ra[i].u;
    }
#pragma unroll
    for (int i = 0; i < B_PT; ++i) {
      const int q = tid + i * NT;
      lds_b[buf * BN * kLdsStride + (q >> 2) * kLdsStride + (q & 3)] = rb[i].u;
    }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;
  auto compute = [&](int buf) {
    const uint4* la = lds_a + buf * BM * kLdsStride;
    const uint4* lb = lds_b + buf * BN * kLdsStride;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Chunk fa[TM], fb[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) fa[tm].u = la[((wm * TM + tm) * 32 + frag_row) * kLdsStride + 2 * j + frag_half];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) fb[tn].u = lb[((wn * TN + tn) * 32 + frag_row) * kLdsStride + 2 * j + frag_half];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) mma<T>(fb[tn], fa[tm], acc[tm][tn]);
    }
  };

  // Register set 0 carries the even tiles, set 1 the odd ones.  The loop has no
  // conditionals: tiles past the end of the reduction load as zeros (out-of-range
  // buffer offsets) and multiply to nothing, so an odd tile count costs one empty step.
  load_tiles(0, ra0, rb0);
  load_tiles(1, ra1, rb1);
  store_tiles(0, ra0, rb0);
  __syncthreads();
  load_tiles(2, ra0, rb0);
  for (int kt = 0; kt < nk; kt += 2) {
    compute(0);  // tile kt
    store_tiles(1, ra1, rb1);
    __syncthreads();
    load_tiles(kt + 3, ra1, rb1);
    compute(1);  // tile kt + 1
    store_tiles(0, ra0, rb0);
    __syncthreads();
    load_tiles(kt + 4, ra0, rb0);
  }

  finish_tile<T, MODE, WM, WN, TM, TN>(p, acc, reinterpret_cast<float*>(lds), tid, m0, n0, tile_m);
}

// ---------------------------------------------------------------------------
// weight gradient
// ---------------------------------------------------------------------------
// `id`: the workgroup's place among the tiles_m * tiles_n * splits workgroups of this weight gradient
template <typename T, int WM, int WN, int TM, int TN>
__device__ __forceinline__ void wgrad_body(const IgemmArgs& p, uint32_t id) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int BKP = 4 * E;  // pixels per reduction step
  constexpr int BM = WM * TM * 32;
  constexpr int BN = WN * TN * 32;
  constexpr int NT = WM * WN * 64;
  constexpr int EB = sizeof(T);
  constexpr int CA = BM / E, CB = BN / E;        // data chunks per [pixel] row
  constexpr int LDA = CA + kRowPad, LDB = CB + kRowPad;  // row stride in chunks
  constexpr int A_PT = (BKP * CA) / NT;
  constexpr int B_PT = (BKP * CB) / NT;
  static_assert((BKP * CA) % NT == 0 && (BKP * CB) % NT == 0, "tile/loader mismatch");
  static_assert(NT % CA == 0 && NT % CB == 0, "a thread keeps one chunk column");
  constexpr int OPER_BYTES = 2 * BKP * (LDA + LDB) * 16;
  constexpr int STAGE_BYTES = WM * 32 * (BN + kStagePad) * 4;
  constexpr int LDS_BYTES = OPER_BYTES > STAGE_BYTES ? OPER_BYTES : STAGE_BYTES;

  __shared__ uint4 lds[LDS_BYTES / 16];
  uint4* lds_a = lds;                      // [2][BKP][LDA]
  uint4* lds_b = lds + 2 * BKP * LDA;      // [2][BKP][LDB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  const int tiles_mn = p.tiles_m * p.tiles_n;
  const int split = id / tiles_mn;
  id -= split * tiles_mn;
  const int tile_m = id / p.tiles_n;
  const int tile_n = id - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int k_begin = split * p.k_per_split;
  int k_end = k_begin + p.k_per_split;
  if (k_end > p.gemm_k) k_end = p.gemm_k;
  const int nk = (k_end - k_begin + BKP - 1) / BKP;

  // operand A = dy[pixel][K]: this thread's channel chunk and first pixel row
  const int a_cc = tid % CA, a_prow = tid / CA;
  const int a_ch = m0 + a_cc * E;
  const bool a_ch_ok = a_ch < p.gemm_m;
  // operand B = x gathered: column n = (tap, channel) is fixed per thread
  const int b_cc = tid % CB, b_prow = tid / CB;
  const int b_n = n0 + b_cc * E;
  const bool b_n_ok = b_n < p.gemm_n;
  int b_r = 0, b_s = 0, b_c = 0;
  if (b_n_ok) {
    const int tap = b_n / p.C;
    b_c = b_n - tap * p.C;
    b_r = tap / p.S;
    b_s = tap - b_r * p.S;
  }

  Chunk ra0[A_PT], rb0[B_PT], ra1[A_PT], rb1[B_PT];
  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a_src, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b_src, p.b_bytes);

  auto load_tiles = [&](int kt, Chunk* ra, Chunk* rb) {
    const int k0 = k_begin + kt * BKP;
#pragma unroll
    for (int i = 0; i < A_PT; ++i) {
      const int pix = k0 + a_prow + i * (NT / CA);
      ra[i] = load_chunk(rsrc_a, static_cast<uint32_t>(pix * p.K + a_ch) * EB, a_ch_ok && pix < k_end);
    }
#pragma unroll
    for (int i = 0; i < B_PT; ++i) {
      const int pix = k0 + b_prow + i * (NT / CB);
      bool ok = b_n_ok && pix < k_end;
      uint32_t off;
      if (p.pointwise) {
        off = static_cast<uint32_t>(pix * p.C + b_c) * EB;
      } else {
        uint32_t img, rem, oh, ow;
        p.div_plane.divmod(static_cast<uint32_t>(pix), img, rem);
        p.div_width.divmod(rem, oh, ow);
        const int hi = static_cast<int>(oh) * p.stride - p.pad + b_r;
        const int wi = static_cast<int>(ow) * p.stride - p.pad + b_s;
        ok = ok && static_cast<unsigned>(hi) < static_cast<unsigned>(p.H) &&
             static_cast<unsigned>(wi) < static_cast<unsigned>(p.W);
        off = static_cast<uint32_t>((static_cast<int>(img) * p.H * p.W + hi * p.W + wi) * p.C + b_c) * EB;
      }
      rb[i] = load_chunk(rsrc_b, off, ok);
    }
  };

  // The bias gradient of a linear layer is the column sum of dy: the workgroups of the first column tile add
  // up the dy chunks they stage anyway (every pixel of the split passes through exactly once).
  const bool sum_dy = p.dbias != nullptr && tile_n == 0;
  float bsum[E];
#pragma unroll
  for (int e = 0; e < E; ++e) bsum[e] = 0.f;

  auto store_tiles = [&](int buf, const Chunk* ra, const Chunk* rb) {
#pragma unroll
    for (int i = 0; i < A_PT; ++i) lds_a[(buf * BKP + a_prow + i * (NT / CA)) * LDA + a_cc] = ra[i].u;
#pragma unroll
    for (int i = 0; i < B_PT; ++i) lds_b[(buf * BKP + b_prow + i * (NT / CB)) * LDB + b_cc] = rb[i].u;
    if (sum_dy) {
#pragma unroll
      for (int i = 0; i < A_PT; ++i) {
        float v[E];
        chunk_to_float<T>(ra[i], v);
#pragma unroll
        for (int e = 0; e < E; ++e) bsum[e] += v[e];
      }
    }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;


  // transpose-read geometry (bf16): lane = 16*G + q; the 16 lanes of a group read
  // pixels {base + q/4 ...} x channels {16*(G%2) + 4*(q%4) ...}; after the transpose
  // lane q owns channel 16*(G%2) + q of the band and 4 pixels.
  const int grp = lane >> 4, q16 = lane & 15;
  const int tr_pix = 8 * (grp >> 1) + (q16 >> 2);
  const int tr_ch = 16 * (grp & 1) + 4 * (q16 & 3);

  auto compute = [&](int buf) {
    if constexpr (sizeof(T) == 2) {
      const uint16_t* la = reinterpret_cast<const uint16_t*>(lds_a + buf * BKP * LDA);
      const uint16_t* lb = reinterpret_cast<const uint16_t*>(lds_b + buf * BKP * LDB);
#pragma unroll
      for (int ks = 0; ks < BKP / 16; ++ks) {
        Chunk fa[TM], fb[TN];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int prow = ks * 16 + tr_pix + 4 * t;
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            const uint16_t* ptr = la + prow * (LDA * 8) + (wm * TM + tm) * 32 + tr_ch;
            TrPart v;
            v.s = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(ptr));
            fa[tm].w[2 * t] = v.w[0];
            fa[tm].w[2 * t + 1] = v.w[1];
          }
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) {
            const uint16_t* ptr = lb + prow * (LDB * 8) + (wn * TN + tn) * 32 + tr_ch;
            TrPart v;
            v.s = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(ptr));
            fb[tn].w[2 * t] = v.w[0];
            fb[tn].w[2 * t + 1] = v.w[1];
          }
        }
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) mma<T>(fb[tn], fa[tm], acc[tm][tn]);
      }
    } else {
      // fp32: one reduction element per lane and MFMA, no transposition needed
      const float* la = reinterpret_cast<const float*>(lds_a + buf * BKP * LDA);
      const float* lb = reinterpret_cast<const float*>(lds_b + buf * BKP * LDB);
#pragma unroll
      for (int ks = 0; ks < BKP / 2; ++ks) {
        const int prow = ks * 2 + (lane >> 5);
        float fa[TM], fb[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) fa[tm] = la[prow * (LDA * 4) + (wm * TM + tm) * 32 + (lane & 31)];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) fb[tn] = lb[prow * (LDB * 4) + (wn * TN + tn) * 32 + (lane & 31)];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[tn], fa[tm], acc[tm][tn], 0, 0, 0);
      }
    }
  };

  // Register set 0 carries the even tiles, set 1 the odd ones.  The loop has no
  // conditionals: tiles past the end of the reduction load as zeros (out-of-range
  // buffer offsets) and multiply to nothing, so an odd tile count costs one empty step.
  load_tiles(0, ra0, rb0);
  load_tiles(1, ra1, rb1);
  store_tiles(0, ra0, rb0);
  __syncthreads();
  load_tiles(2, ra0, rb0);
  for (int kt = 0; kt < nk; kt += 2) {
    compute(0);  // tile kt
    store_tiles(1, ra1, rb1);
    __syncthreads();
    load_tiles(kt + 3, ra1, rb1);
    compute(1);  // tile kt + 1
    store_tiles(0, ra0, rb0);
    __syncthreads();
    load_tiles(kt + 4, ra0, rb0);
  }


  float* out = static_cast<float*>(p.out);
  if (p.splits > 1) out += static_cast<int64_t>(split) * p.gemm_m * p.gemm_n;
  const bool accumulate = p.splits == 1 && p.accumulate;
  staged_epilogue<T, WM, WN, TM, TN>(acc, reinterpret_cast<float*>(lds), tid, [&](int, int tr, int tc, float* v) {
    const int row = m0 + tr, col = n0 + tc;
    if (row >= p.gemm_m || col >= p.gemm_n) return;
    float* dst = out + static_cast<int64_t>(row) * p.gemm_n + col;
    if (accumulate) {
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] += dst[e];
    }
    store_floats<E>(dst, v);
  });
  if (sum_dy) {
    // NT / CA threads hold partial sums of the same E channels: through LDS, then one thread per channel
    float* red = reinterpret_cast<float*>(lds);
    __syncthreads();
#pragma unroll
    for (int e = 0; e < E; ++e) red[a_prow * BM + a_cc * E + e] = bsum[e];
    __syncthreads();
    if (tid < BM && m0 + tid < p.gemm_m) {
      float s = 0.f;
#pragma unroll
      for (int r = 0; r < NT / CA; ++r) s += red[r * BM + tid];
      float* dst = p.dbias + (p.splits > 1 ? static_cast<int64_t>(split) * p.gemm_m : 0) + m0 + tid;
      *dst = accumulate ? *dst + s : s;
    }
  }
}

__device__ __forceinline__ void splitk_reduce_body(const ReduceArgs& p, uint32_t block);

// One weight gradient, and optionally -- as the workgroups from gemm_wgs on -- the split reduction of the weight
// gradient launched BEFORE it on the same stream: its partials are complete by stream order, so the reduction needs no
// launch of its own and runs beside this gradient's multiplications instead of behind them.
struct WgradArgs {
  IgemmArgs a;
  ReduceArgs red;      // red.n == 0: nothing rides along
  uint32_t gemm_wgs;
};

template <typename T, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM* WN * 64) void wgrad_kernel(WgradArgs w) {
  if (blockIdx.x >= w.gemm_wgs) {
    splitk_reduce_body(w.red, blockIdx.x - w.gemm_wgs);
    return;
  }
  wgrad_body<T, WM, WN, TM, TN>(w.a, xcd_remap(blockIdx.x, w.gemm_wgs));
}

// The weight gradients of several convolutions in one launch.  `table` holds one argument block per convolution,
// `map` one entry per workgroup: (which convolution, which of its workgroups).  Neighbouring entries of the map
// are workgroups of the same convolution and split, so that after the XCD remap the workgroups that share
// operand rows also share an L2.  Both arrays are read with wave-uniform addresses.
// With fewer workgroups than entries a workgroup takes every gridDim.x-th entry: a launch that is meant to run
// beside other kernels for a long time on a share of every CU instead of flooding the chip.
struct WgradGroupArgs {
  const IgemmArgs* table;
  const uint2* map;
  uint32_t entries;
};

template <typename T, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM* WN * 64) void wgrad_group_kernel(WgradGroupArgs g) {
  for (uint32_t gid = xcd_remap(blockIdx.x, gridDim.x); gid < g.entries; gid += gridDim.x) {
    const uint2 e = g.map[gid];
    const IgemmArgs p = g.table[__builtin_amdgcn_readfirstlane(e.x)];
    wgrad_body<T, WM, WN, TM, TN>(p, __builtin_amdgcn_readfirstlane(e.y));
    __syncthreads();   // the next entry's operand tiles overwrite what the epilogue staged in LDS
  }
}

// ---------------------------------------------------------------------------
// forward / data gradient, bf16, channel counts that are multiples of 64
// ---------------------------------------------------------------------------
// Same GEMM view as igemm_kernel, restructured around what gfx950 offers:
//   * operand tiles go from global memory straight into LDS (buffer_load ... lds, 16 bytes
//     per lane, out-of-range offsets land as zeros): no staging registers, no LDS stores;
//   * one reduction step is 64 elements = one 128-byte LDS row per GEMM row, unpadded, with
//     the 16-byte slot index XOR-ed by (row >> 1) & 7 so that a 16-lane group of an MFMA
//     operand read touches every bank once;
//   * a step never straddles a filter tap (channels % 64 == 0), so the tap walk is scalar:
//     a lane keeps one byte offset and one validity bit per tap for each row it loads;
//   * NBUF tiles in flight, one barrier per step;
//   * KS = 32 halves the step (64-byte rows, sixteen rows per direct load): half the LDS per tile in flight, so
//     more workgroups share a CU and a small grid is resident in one round.
constexpr int kStep2 = 64;                  // reduction elements per step
constexpr int kRowBytes2 = kStep2 * 2;      // 128

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// 16 bytes per lane from `rsrc` at byte offset voff (+ the wave-uniform soff) to dst + lane*16 in
// LDS; an offset outside the resource stores zeros.  (Kept in a device function: named directly
// in a kernel body, the builtin makes the host pass drop the kernel's launch stub.)
__device__ inline void load_to_lds(__amdgpu_buffer_rsrc_t rsrc, unsigned char* dst, int voff, int soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)dst, 16, voff, soff, 0, 0);
}

template <int MODE, int WM, int WN, int TM, int TN, int NBUF, int ROT = 0, int KS = kStep2>
__global__ __launch_bounds__(WM* WN * 64) void igemm2_kernel(IgemmArgs p) {
  using T = bf16;
  constexpr int E = 8;
  constexpr int BM = WM * TM * 32;
  constexpr int BN = WN * TN * 32;
  constexpr int NW = WM * WN;
  static_assert(KS == 64 || KS == 32, "reduction elements per step");
  constexpr int RB = KS * 2;             // bytes of one LDS row
  constexpr int SLOTS = RB / 16;         // 16-byte slots per row: 8 or 4
  constexpr int SLOT_SH = KS == 64 ? 3 : 2;
  constexpr int LD_ROWS = 1024 / RB;     // rows one direct load of a wave fills: 8 or 16
  constexpr int A_LD = BM / LD_ROWS / NW;  // direct loads per wave and step for the activation tile
  constexpr int B_LD = BN / LD_ROWS / NW;
  static_assert(BM % (LD_ROWS * NW) == 0 && BN % (LD_ROWS * NW) == 0, "tile/loader mismatch");
  constexpr int A_BYTES = BM * RB, B_BYTES = BN * RB;
  // slot = chunk ^ swizzle(row): with 128-byte rows two rows span the 64 banks and (row >> 1) & 7 spreads sixteen
  // rows of one chunk over all of them; with 64-byte rows four rows span them and (row >> 2) & 3 does the same
  auto swizzle = [](int row) { return KS == 64 ? (row >> 1) & 7 : (row >> 2) & 3; };
  constexpr int BUF_BYTES = A_BYTES + B_BYTES;
  constexpr int STAGE_BYTES = WM * 32 * (BN + kStagePad) * 4;
  constexpr int LDS_BYTES = NBUF * BUF_BYTES > STAGE_BYTES ? NBUF * BUF_BYTES : STAGE_BYTES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  uint32_t id = xcd_remap(blockIdx.x, gridDim.x);
  int tile_m, tile_n;
  if (p.group_rows > 1) {
    // wide outputs: consecutive ids walk down group_rows row tiles before they move one column tile on, so that
    // the tiles an XCD works on at one time form a squarish block (fewer distinct operand rows through its L2)
    const uint32_t per_group = static_cast<uint32_t>(p.group_rows) * p.tiles_n;
    const uint32_t grp = id / per_group;
    const uint32_t local = id - grp * per_group;
    const uint32_t first = grp * p.group_rows;
    const uint32_t rows = min(static_cast<uint32_t>(p.group_rows), static_cast<uint32_t>(p.tiles_m) - first);
    tile_n = local / rows;
    tile_m = first + (local - tile_n * rows);
  } else {
    tile_m = id / p.tiles_n;
    tile_n = id - tile_m * p.tiles_n;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int in_h = (MODE == kFwd) ? p.H : p.Ho;
  const int in_w = (MODE == kFwd) ? p.W : p.Wo;
  const int in_c = (MODE == kFwd) ? p.C : p.K;
  const int cblocks = in_c / KS;
  const int nk = p.R * p.S * cblocks;
  const int sl = p.stride_log2, sm = p.stride - 1;

  // ---- per lane: the rows it feeds, their byte offset at tap (0,0) and which taps exist ----
  const int sub_row = lane >> SLOT_SH, slot = lane & (SLOTS - 1);
  int a_off[A_LD];
  uint32_t a_taps[A_LD];
#pragma unroll
  for (int j = 0; j < A_LD; ++j) {
    const int trow = (wave * A_LD + j) * LD_ROWS + sub_row;
    const int chunk = slot ^ swizzle(trow);
    const int row = m0 + trow;
    uint32_t img = 0, pix = 0, oh = 0, ow = 0, taps = 0;
    int base = 0;
    if (row < p.gemm_m) {
      p.div_plane.divmod(static_cast<uint32_t>(row), img, pix);
      p.div_width.divmod(pix, oh, ow);
      if (MODE == kFwd) {
        const int h0 = static_cast<int>(oh) * p.stride - p.pad, w0 = static_cast<int>(ow) * p.stride - p.pad;
        base = ((static_cast<int>(img) * in_h + h0) * in_w + w0) * in_c;
        for (int r = 0; r < p.R; ++r)
          for (int s = 0; s < p.S; ++s)
            if (static_cast<unsigned>(h0 + r) < static_cast<unsigned>(in_h) &&
                static_cast<unsigned>(w0 + s) < static_cast<unsigned>(in_w))
              taps |= 1u << (r * p.S + s);
      } else {
        const int hp = static_cast<int>(oh) + p.pad, wp = static_cast<int>(ow) + p.pad;
        base = ((static_cast<int>(img) * in_h + (hp >> sl)) * in_w + (wp >> sl)) * in_c;
        for (int r = 0; r < p.R; ++r)
          for (int s = 0; s < p.S; ++s) {
            const int th = hp - r, tw = wp - s;
            if (th >= 0 && tw >= 0 && (th & sm) == 0 && (tw & sm) == 0 && (th >> sl) < in_h && (tw >> sl) < in_w)
              taps |= 1u << (r * p.S + s);
          }
      }
    }
    a_off[j] = (base + chunk * E) * 2;
    a_taps[j] = taps;
  }
  int b_off[B_LD];
#pragma unroll
  for (int j = 0; j < B_LD; ++j) {
    const int trow = (wave * B_LD + j) * LD_ROWS + sub_row;
    const int chunk = slot ^ swizzle(trow);
    const int row = n0 + trow;
    b_off[j] = row < p.gemm_n ? (row * p.gemm_k + chunk * E) * 2 : static_cast<int>(kOutOfRange);
  }

  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a_src, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b_src, p.b_bytes);

  // scalar walk over (tap, channel block)
  int ld_r = 0, ld_s = 0, ld_cb = 0, ld_t = 0, ld_kt = 0;
  auto issue_loads = [&](int buf) {
    // element offset of this tap relative to tap (0,0), then bytes
    const int tap_elems = (MODE == kFwd) ? (ld_r * in_w + ld_s) * in_c : -((ld_r >> sl) * in_w + (ld_s >> sl)) * in_c;
    const int a_step = (tap_elems + ld_cb * KS) * 2;
    const int b_step = ld_kt * RB;
    unsigned char* dst_a = lds + buf * BUF_BYTES + wave * A_LD * 1024;
    unsigned char* dst_b = lds + buf * BUF_BYTES + A_BYTES + wave * B_LD * 1024;
#pragma unroll
    for (int j = 0; j < A_LD; ++j) {
      const bool ok = (a_taps[j] >> ld_t) & 1u;
      const int off = ok ? a_off[j] + a_step : static_cast<int>(kOutOfRange);
      load_to_lds(rsrc_a, dst_a + j * 1024, off, 0);
    }
#pragma unroll
    for (int j = 0; j < B_LD; ++j)
      load_to_lds(rsrc_b, dst_b + j * 1024, b_off[j], b_step);
    ++ld_kt;
    if (++ld_cb == cblocks) {
      ld_cb = 0;
      ++ld_t;
      if (++ld_s == p.S) {
        ld_s = 0;
        ++ld_r;
      }
    }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand reads: row = tile row of the lane, slot = chunk ^ swizzle(row); the tile bases are
  // multiples of 32 rows, so the swizzle term depends on the lane only
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int swz = swizzle(frag_row);
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
  const uint32_t a_rd = lds_base + (wm * TM * 32 + frag_row) * RB + swz * 16;
  const uint32_t b_rd = lds_base + A_BYTES + (wn * TN * 32 + frag_row) * RB + swz * 16;
  // The operand reads are written as asm: the compiler orders every LDS read it can see behind
  // ALL outstanding direct-to-LDS loads (vmcnt(0)), which would serialise the prefetch of the
  // next tiles with the multiply of this one.  Which loads must have landed is known here (the
  // counted wait + barrier at the top of a step), so the reads carry their own lgkmcnt waits.
  auto read_frags = [&](int buf, int kk, uint4_t* fa, uint4_t* fb) {
    const uint32_t cx = (2 * kk + frag_half) * 16;
    const uint32_t pa = (a_rd ^ cx) + buf * BUF_BYTES, pb = (b_rd ^ cx) + buf * BUF_BYTES;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[tm]) : "v"(pa), "n"(tm * 32 * RB));
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[tn]) : "v"(pb), "n"(tn * 32 * RB));
  };
  auto multiply = [&](uint4_t* fa, uint4_t* fb) {
    // ties the registers to the wait that precedes this call in program order
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) asm volatile("" : "+v"(fa[tm]));
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) asm volatile("" : "+v"(fb[tn]));
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fb[tn]),
                                                              __builtin_bit_cast(bf16x8_t, fa[tm]), acc[tm][tn], 0, 0, 0);
  };
  auto compute = [&](int buf) {
    uint4_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    read_frags(buf, 0, fa0, fb0);
    read_frags(buf, 1, fa1, fb1);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa0, fb0);
    if constexpr (KS == 32) {   // a 32-element step holds two 16-element slices
      asm volatile("s_waitcnt lgkmcnt(0)");
      multiply(fa1, fb1);
      return;
    }
    read_frags(buf, 2, fa0, fb0);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa1, fb1);
    read_frags(buf, 3, fa1, fb1);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa0, fb0);
    asm volatile("s_waitcnt lgkmcnt(0)");
    multiply(fa1, fb1);
  };

  // vmcnt(n): at most n of this wave's loads still in flight (gfx9 encoding, nothing else waited for)
  constexpr int LOADS = A_LD + B_LD;
  constexpr int AHEAD = (NBUF - 2) * LOADS;
  constexpr int WAIT_IMM = (AHEAD & 0xF) | ((AHEAD >> 4) << 14) | (0x7 << 4) | (0xF << 8);
  static_assert(AHEAD < 64, "vmcnt range");

  // One step = wait until only the newer tiles' loads are outstanding (then this wave's part of tile kt has
  // landed; near the end fewer newer tiles exist, so wait for everything), barrier (every wave's part is in
  // LDS and every wave is done with tile kt-1), request the tile NBUF-1 steps ahead into the buffer that just
  // became free, multiply.  The main loop takes NBUF steps per trip with the buffer index a constant and the
  // multiply outside every conditional (inside one, the compiler moves the 64 accumulators between register
  // classes in every step); the last nk % NBUF steps follow one by one.
  auto step = [&](int kt, int u) {
    if (kt + NBUF - 1 <= nk)
      __builtin_amdgcn_s_waitcnt(WAIT_IMM);
    else
      __builtin_amdgcn_s_waitcnt((0x7 << 4) | (0xF << 8));
    __syncthreads();
    if (kt + NBUF - 1 < nk) issue_loads((u + NBUF - 1) % NBUF);
    compute(u);
  };
  if constexpr (ROT) {
    // Rotated loop for the large tiles, whose workgroup has a compute unit to itself (nobody else fills the
    // gap a barrier leaves): the barrier that hands over tile kt+1 sits BEFORE the last quarter of tile kt's
    // multiplies, whose operands are in registers by then, and the first operand reads of tile kt+1 are issued
    // in front of that quarter.  The matrix pipeline therefore has a quarter's multiplies to chew on while the
    // barrier, the reads' latency and the issue of the next tile's loads pass.  Every wait stands behind a
    // quarter's multiplies that were issued after the reads it waits for, and nothing is in flight at the loop
    // edge.  Order of additions per accumulator: as in the plain loop (same results bit for bit).
    static_assert(NBUF == 2 && KS == 64, "the rotated loop keeps two 64-element tiles in LDS");
    uint4_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    issue_loads(0);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    if (1 < nk) issue_loads(1);
    read_frags(0, 0, fa0, fb0);
    asm volatile("s_waitcnt lgkmcnt(0)");
    auto body = [&](int kt, int u) {
      read_frags(u, 1, fa1, fb1);
      multiply(fa0, fb0);
      asm volatile("s_waitcnt lgkmcnt(0)");
      read_frags(u, 2, fa0, fb0);
      multiply(fa1, fb1);
      asm volatile("s_waitcnt lgkmcnt(0)");
      read_frags(u, 3, fa1, fb1);
      multiply(fa0, fb0);
      // all of tile kt is in registers; tile kt+1 (the only loads outstanding) must have landed
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (kt + 1 < nk) read_frags(u ^ 1, 0, fa0, fb0);
      multiply(fa1, fb1);
      if (kt + 2 < nk) issue_loads(u);
      asm volatile("s_waitcnt lgkmcnt(0)");
    };
    int kt0 = 0;
    for (; kt0 + 2 <= nk; kt0 += 2) {
      body(kt0, 0);
      body(kt0 + 1, 1);
    }
    if (kt0 < nk) body(kt0, 0);
    __syncthreads();   // the epilogue stages through the operand buffers: every wave is done reading them
  } else {
#pragma unroll
    for (int s = 0; s < NBUF - 1; ++s)
      if (s < nk) issue_loads(s);
    int kt0 = 0;
    for (; kt0 + NBUF <= nk; kt0 += NBUF) {
#pragma unroll
      for (int u = 0; u < NBUF; ++u) step(kt0 + u, u);
    }
#pragma unroll
    for (int u = 0; u < NBUF - 1; ++u)
      if (kt0 + u < nk) step(kt0 + u, u);
  }

  finish_tile<T, MODE, WM, WN, TM, TN>(p, acc, reinterpret_cast<float*>(lds), tid, m0, n0, tile_m);
}

// ---------------------------------------------------------------------------
// 3x3, stride 1, pad 1 (forward and data gradient), 128 x 64*TN tile: the activation side of the nine
// taps of a channel block is ONE patch in LDS.  The 128 output pixels of a tile are consecutive in the
// flattened (image, row, column) order, and the input pixel of tap (r, s) lies (r-1)*W + (s-1) places
// further in the same order, so the patch is the contiguous range of pixels from W+1 before the tile to
// W+1 behind it (128 + 2W + 2 rows of 64 channels), loaded once per channel block instead of nine
// shifted copies of the tile.  A tap that falls outside its image (the zero padding) reads a row of
// zeros kept in LDS instead.  The filter tiles stream per (channel block, tap) as in igemm2_kernel,
// three in flight; the patch of the next channel block is requested at the first tap of this one.
// The reduction runs channel block by channel block (taps innermost), so sums round differently from
// igemm2_kernel's tap-major order.
// ---------------------------------------------------------------------------
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

template <int MODE, int TN, int NBUF, int P_LD>
__global__ __launch_bounds__(256) void igemm3_kernel(IgemmArgs p) {
  using T = bf16;
  constexpr int E = 8, WM = 2, WN = 2, TM = 2, NW = 4;
  static_assert(NBUF >= 2 && NBUF <= 4, "filter tiles in flight");
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int B_LD = BN / 8 / NW;
  constexpr int PATCH_BYTES = P_LD * 32 * kRowBytes2, B_BYTES = BN * kRowBytes2;
  constexpr int B_OFF = 2 * PATCH_BYTES, ZERO_OFF = B_OFF + NBUF * B_BYTES;
  constexpr int STAGE_BYTES = WM * 32 * (BN + kStagePad) * 4;
  constexpr int LDS_BYTES = ZERO_OFF + kRowBytes2 > STAGE_BYTES ? ZERO_OFF + kRowBytes2 : STAGE_BYTES;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  uint32_t id = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = id / p.tiles_n;
  const int tile_n = id - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int in_c = (MODE == kFwd) ? p.C : p.K;
  const int cblocks = in_c / kStep2;
  const int nk = 9 * cblocks;
  const int W = p.W, H = p.H, halo = W + 1;

  // ---- loaders: patch rows (wave * P_LD + j) * 8 + lane / 8, filter rows as in igemm2_kernel ----
  const int sub_row = lane >> 3, slot = lane & 7;
  int p_off[P_LD];
#pragma unroll
  for (int j = 0; j < P_LD; ++j) {
    const int prow = (wave * P_LD + j) * 8 + sub_row;
    const int chunk = slot ^ ((prow >> 1) & 7);
    const int grow = m0 - halo + prow;
    const bool ok = grow >= 0 && grow < p.gemm_m && prow < BM + 2 * halo;
    p_off[j] = ok ? (grow * in_c + chunk * E) * 2 : static_cast<int>(kOutOfRange);
  }
  int b_off[B_LD];
#pragma unroll
  for (int j = 0; j < B_LD; ++j) {
    const int trow = (wave * B_LD + j) * 8 + sub_row;
    const int chunk = slot ^ ((trow >> 1) & 7);
    const int row = n0 + trow;
    b_off[j] = row < p.gemm_n ? (row * p.gemm_k + chunk * E) * 2 : static_cast<int>(kOutOfRange);
  }
  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a_src, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b_src, p.b_bytes);
  auto issue_patch = [&](int cb) {
    unsigned char* dst = lds + (cb & 1) * PATCH_BYTES + wave * P_LD * 1024;
#pragma unroll
    for (int j = 0; j < P_LD; ++j) load_to_lds(rsrc_a, dst + j * 1024, p_off[j], cb * kRowBytes2);
  };
  auto issue_filter = [&](int cb, int tap, int buf) {
    unsigned char* dst = lds + B_OFF + buf * B_BYTES + wave * B_LD * 1024;
    const int soff = (tap * in_c + cb * kStep2) * 2;
#pragma unroll
    for (int j = 0; j < B_LD; ++j) load_to_lds(rsrc_b, dst + j * 1024, b_off[j], soff);
  };

  // ---- the rows this lane feeds to the MFMAs and which of their nine taps lie inside the image ----
  const int frag_row = lane & 31, frag_half = lane >> 5;
  uint32_t taps[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int row = m0 + (wm * TM + tm) * 32 + frag_row;
    uint32_t bits = 0;
    if (row < p.gemm_m) {
      uint32_t img, pix, oh, ow;
      p.div_plane.divmod(static_cast<uint32_t>(row), img, pix);
      p.div_width.divmod(pix, oh, ow);
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s2 = 0; s2 < 3; ++s2) {
          const int ih = (MODE == kFwd) ? static_cast<int>(oh) + r - 1 : static_cast<int>(oh) + 1 - r;
          const int iw = (MODE == kFwd) ? static_cast<int>(ow) + s2 - 1 : static_cast<int>(ow) + 1 - s2;
          if (static_cast<unsigned>(ih) < static_cast<unsigned>(H) && static_cast<unsigned>(iw) < static_cast<unsigned>(W))
            bits |= 1u << (r * 3 + s2);
        }
    }
    taps[tm] = bits;
  }

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
  const int swz = (frag_row >> 1) & 7;
  const uint32_t b_rd = lds_base + B_OFF + (wn * TN * 32 + frag_row) * kRowBytes2 + swz * 16;

  // One step = one (channel block, tap).  pa[tm]: LDS address of this lane's patch row for the tap (slot
  // swizzle of that row included), or of the zero row.
  auto compute = [&](uint32_t patch_base, int tap, int buf) {
    const int r = tap / 3, s2 = tap - 3 * r;
    const int tapoff = (MODE == kFwd) ? r * W + s2 : (2 - r) * W + (2 - s2);
    uint32_t pa[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const uint32_t prow = static_cast<uint32_t>((wm * TM + tm) * 32 + frag_row + tapoff);
      const uint32_t in_patch = patch_base + prow * kRowBytes2 + ((prow >> 1) & 7) * 16;
      pa[tm] = ((taps[tm] >> tap) & 1u) ? in_patch : lds_base + ZERO_OFF;
    }
    const uint32_t pb0 = b_rd + buf * B_BYTES;
    auto read_frags = [&](int kk, uint4_t* fa, uint4_t* fb) {
      const uint32_t cx = (2 * kk + frag_half) * 16;
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) asm volatile("ds_read_b128 %0, %1" : "=v"(fa[tm]) : "v"(pa[tm] ^ cx));
      const uint32_t pb = pb0 ^ cx;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[tn]) : "v"(pb), "n"(tn * 32 * kRowBytes2));
    };
    auto multiply = [&](uint4_t* fa, uint4_t* fb) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) asm volatile("" : "+v"(fa[tm]));
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) asm volatile("" : "+v"(fb[tn]));
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fb[tn]),
                                                                __builtin_bit_cast(bf16x8_t, fa[tm]), acc[tm][tn], 0, 0, 0);
    };
    uint4_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    read_frags(0, fa0, fb0);
    read_frags(1, fa1, fb1);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa0, fb0);
    read_frags(2, fa0, fb0);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa1, fb1);
    read_frags(3, fa1, fb1);
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
    multiply(fa0, fb0);
    asm volatile("s_waitcnt lgkmcnt(0)");
    multiply(fa1, fb1);
  };

  // Requests leave in this order: patch 0, filters 0 .. NBUF-2; then at step kt, behind its barrier, filter
  // kt + NBUF-1 (into the buffer step kt-1 read) and, at the first tap of a channel block, the next block's
  // patch.  They land in order, so "filter kt has landed" (and every patch requested before it) is a count
  // of the requests made after it: the NBUF-2 filters behind it, and the patch requested at tap 0 when this
  // is one of the taps 1 .. NBUF-1.  (Over the last steps fewer filters follow: wait for everything.)
  constexpr int AHEAD = NBUF - 1;
  if (tid < 8) *reinterpret_cast<uint4*>(lds + ZERO_OFF + tid * 16) = make_uint4(0u, 0u, 0u, 0u);
  issue_patch(0);
#pragma unroll
  for (int t = 0; t < AHEAD; ++t) issue_filter(0, t, t);
  for (int cb = 0; cb < cblocks; ++cb) {
    const uint32_t patch_base = lds_base + (cb & 1) * PATCH_BYTES;
    const bool next_patch = cb + 1 < cblocks;
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      const int kt = cb * 9 + tap;
      if (kt + AHEAD > nk)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
      else if (tap >= 1 && tap <= AHEAD && next_patch)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((NBUF - 2) * B_LD + P_LD));
      else
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((NBUF - 2) * B_LD));
      __syncthreads();
      // 9 taps per channel block: with three buffers the buffer of a step is a constant of the unrolled loop
      const int buf = NBUF == 3 ? tap % 3 : kt % NBUF;
      const int buf_ahead = NBUF == 3 ? (tap + AHEAD) % 3 : (kt + AHEAD) % NBUF;
      if (kt + AHEAD < nk) issue_filter(tap + AHEAD >= 9 ? cb + 1 : cb, (tap + AHEAD) % 9, buf_ahead);
      if (tap == 0 && next_patch) issue_patch(cb + 1);
      compute(patch_base, tap, buf);
    }
  }

  finish_tile<T, MODE, WM, WN, TM, TN>(p, acc, reinterpret_cast<float*>(lds), tid, m0, n0, tile_m);
}

__device__ __forceinline__ void splitk_reduce_body(const ReduceArgs& p, uint32_t block) {
  if (block >= p.first_blocks) {
    const int i = (block - p.first_blocks) * 256 + threadIdx.x;
    if (i >= p.n2) return;
    float s = 0.f;
    constexpr int U2 = 8;
    for (int k0 = 0; k0 < p.splits; k0 += U2) {
      float v[U2];
#pragma unroll
      for (int u = 0; u < U2; ++u) v[u] = p.partial2[static_cast<int64_t>(k0 + u < p.splits ? k0 + u : p.splits - 1) * p.n2 + i];
#pragma unroll
      for (int u = 0; u < U2; ++u)
        if (k0 + u < p.splits) s += v[u];
    }
    p.out2[i] = p.accumulate ? p.out2[i] + s : s;
    return;
  }
  int64_t i = (static_cast<int64_t>(block) * 256 + threadIdx.x) * 4;
  if (i >= p.n) return;
  // Eight partials are requested before any is added (a request past the last split repeats it and does not
  // count): the kernel costs its dependent round trips to memory, one per trip here instead of one per split.
  // The additions keep the order of the splits.
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  constexpr int U = 8;
  for (int k0 = 0; k0 < p.splits; k0 += U) {
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u < p.splits ? k0 + u : p.splits - 1;
      v[u] = *reinterpret_cast<const float4*>(p.partial + static_cast<int64_t>(k) * p.n + i);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (k0 + u < p.splits) {
        s.x += v[u].x;
        s.y += v[u].y;
        s.z += v[u].z;
        s.w += v[u].w;
      }
  }
  float4* o = reinterpret_cast<float4*>(p.out + i);
  if (p.accumulate) {
    float4 c = *o;
    s.x += c.x;
    s.y += c.y;
    s.z += c.z;
    s.w += c.w;
  }
  *o = s;
}

__global__ __launch_bounds__(256) void splitk_reduce_kernel(ReduceArgs p) { splitk_reduce_body(p, blockIdx.x); }

// The split reductions of several weight gradients in one launch (table / map as in wgrad_group_kernel).
struct ReduceGroupArgs {
  const ReduceArgs* table;
  const uint2* map;
};

__global__ __launch_bounds__(256) void splitk_reduce_group_kernel(ReduceGroupArgs g) {
  const uint2 e = g.map[blockIdx.x];
  const ReduceArgs p = g.table[__builtin_amdgcn_readfirstlane(e.x)];
  splitk_reduce_body(p, __builtin_amdgcn_readfirstlane(e.y));
}

int ilog2_exact(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return ((1 << l) == v) ? l : -1;
}

template <typename T, int MODE, int WM, int WN, int TM, int TN>
const char* igemm_name() {
  static const std::string name = std::string(MODE == kWgrad ? "wgrad_kernel<" : "igemm_kernel<") +
                                  (sizeof(T) == 2 ? "bf16" : "f32") + "," +
                                  (MODE == kFwd ? "fwd," : MODE == kDgrad ? "dgrad," : "") +
                                  std::to_string(WM * TM * 32) + "x" + std::to_string(WN * TN * 32) + ">";
  return name.c_str();
}

// Algorithmic bytes of one convolution launch: each operand read once, the result written once (the partial
// results of a split reduction are the kernel's own choice and do not count).  Many of these layers do fewer
// flops per byte than the chip can feed, so the profiler is told the bytes beside the flops.
template <int MODE>
double conv_bytes(const IgemmArgs& a, int eb) {
  const double x = static_cast<double>(a.N) * a.H * a.W * a.C, y = static_cast<double>(a.N) * a.Ho * a.Wo * a.K;
  const double w = static_cast<double>(a.K) * a.R * a.S * a.C;
  if (MODE == kWgrad) return (x + y) * eb + w * 4;
  const double out = MODE == kFwd ? y : x;
  const int extra = (a.add ? 1 : 0) + (a.add && a.mask ? 1 : 0) + (a.bn_x ? 1 : 0) + (a.bn_mask ? 1 : 0);
  return ((MODE == kFwd ? x : y) + w + out * extra) * eb + out * (a.out_f32 ? 4 : eb);
}

template <typename T, int MODE, int WM, int WN, int TM, int TN>
int launch_cfg(Context* ctx, IgemmArgs& a, double flops) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  a.tiles_m = (a.gemm_m + BM - 1) / BM;
  a.tiles_n = (a.gemm_n + BN - 1) / BN;
  int64_t wgs = static_cast<int64_t>(a.tiles_m) * a.tiles_n * a.splits;
  if (wgs <= 0 || wgs > 0x7fffffff) {
    set_error("igemm: grid out of range");
    return -22;
  }
  const dim3 grid(static_cast<unsigned>(wgs)), block(WM * WN * 64);
  if constexpr (MODE == kWgrad) {
    static_assert(WM * WN * 64 == 256, "the split reduction that may ride along is written for 256 threads");
    WgradArgs w{};
    w.a = a;
    w.gemm_wgs = static_cast<uint32_t>(wgs);
    double bytes = conv_bytes<MODE>(a, sizeof(T));
    auto& tr = ctx->trailing_reduce;
    unsigned blocks = grid.x;
    if (a.take_pending && tr.valid) {
      // the launch keeps its own algorithmic bytes (operands once, the filter gradient once): the partial filters
      // the extra workgroups read are traffic, not work
      w.red = tr.args;
      blocks += tr.blocks;
      tr.valid = false;
    }
    return launch(ctx, wgrad_kernel<T, WM, WN, TM, TN>, dim3(blocks), block, w, igemm_name<T, MODE, WM, WN, TM, TN>(), flops, 0,
                  bytes);
  } else
    return launch(ctx, igemm_kernel<T, MODE, WM, WN, TM, TN>, grid, block, a, igemm_name<T, MODE, WM, WN, TM, TN>(),
                  flops, 0, conv_bytes<MODE>(a, sizeof(T)));
}

template <int MODE, int WM, int WN, int TM, int TN, int NBUF, int ROT = 0, int KS = kStep2>
int launch_cfg2(Context* ctx, IgemmArgs& a, double flops) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  static const std::string name = std::string("igemm2_kernel<bf16,") + (MODE == kFwd ? "fwd," : "dgrad,") +
                                  std::to_string(BM) + "x" + std::to_string(BN) + "," + std::to_string(NBUF) + "buf" +
                                  (WM * WN == 8 ? ",8w" : "") + (KS == 32 ? ",k32" : "") + (ROT ? ",rot>" : ">");
  a.tiles_m = (a.gemm_m + BM - 1) / BM;
  a.tiles_n = (a.gemm_n + BN - 1) / BN;
  static const int group_env = [] {
    const char* e = getenv("TCH_IGEMM_GROUP_ROWS");
    return e ? atoi(e) : -1;
  }();
  a.group_rows = group_env >= 0 ? group_env : (a.tiles_n > 8 ? 4 : 0);
  int64_t wgs = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
  if (wgs <= 0 || wgs > 0x7fffffff) {
    set_error("igemm: grid out of range");
    return -22;
  }
  return launch(ctx, igemm2_kernel<MODE, WM, WN, TM, TN, NBUF, ROT, KS>, dim3(static_cast<unsigned>(wgs)), dim3(WM * WN * 64), a,
                name.c_str(), flops, 0, conv_bytes<MODE>(a, 2));
}

// The 3x3 patch kernel: stride 1, pad 1, input channels in blocks of 64, rows short enough for the patch
template <int MODE>
bool patch_kernel_fits(const IgemmArgs& a) {
  const int in_c = MODE == kFwd ? a.C : a.K;
  return a.R == 3 && a.S == 3 && a.stride == 1 && a.pad == 1 && a.H == a.Ho && a.W == a.Wo && in_c % kStep2 == 0 &&
         128 + 2 * (a.W + 1) <= 256;
}

template <int MODE, int TN, int NBUF, int P_LD>
int launch_cfg3_rows(Context* ctx, IgemmArgs& a, double flops) {
  constexpr int BM = 128, BN = 64 * TN;
  static const std::string name = std::string("igemm3_kernel<bf16,") + (MODE == kFwd ? "fwd," : "dgrad,") +
                                  std::to_string(BM) + "x" + std::to_string(BN) + "," + std::to_string(NBUF) + "buf,patch" +
                                  std::to_string(P_LD * 32) + ">";
  a.tiles_m = (a.gemm_m + BM - 1) / BM;
  a.tiles_n = (a.gemm_n + BN - 1) / BN;
  const int64_t wgs = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
  if (wgs <= 0 || wgs > 0x7fffffff) {
    set_error("igemm: grid out of range");
    return -22;
  }
  return launch(ctx, igemm3_kernel<MODE, TN, NBUF, P_LD>, dim3(static_cast<unsigned>(wgs)), dim3(256), a, name.c_str(), flops, 0,
                conv_bytes<MODE>(a, 2));
}

template <int MODE, int TN, int NBUF>
int launch_cfg3(Context* ctx, IgemmArgs& a, double flops) {
  const int rows = 128 + 2 * (a.W + 1);   // patch rows, loaded 32 at a time
  if (rows <= 160) return launch_cfg3_rows<MODE, TN, NBUF, 5>(ctx, a, flops);
  if (rows <= 192) return launch_cfg3_rows<MODE, TN, NBUF, 6>(ctx, a, flops);
  return launch_cfg3_rows<MODE, TN, NBUF, 8>(ctx, a, flops);
}

// TCH_IGEMM2 = 0 keeps every convolution on igemm_kernel; 2 or 3 picks the number of LDS tiles
// in flight of igemm2_kernel (default: 2 for 128x128, 3 for 128x64)
int igemm2_setting() {
  static const int v = [] {
    const char* e = getenv("TCH_IGEMM2");
    return e ? atoi(e) : -1;
  }();
  return v;
}

template <typename T, int MODE>
int launch_mode(Context* ctx, IgemmArgs& a, int tile_cfg, double flops) {
  if constexpr (sizeof(T) == 2 && (MODE == kFwd || MODE == kDgrad)) {
    const int in_c = MODE == kFwd ? a.C : a.K;
    const int setting = igemm2_setting();
    if (tile_cfg == 5) {   // 128 x 64 with the 3x3 patch in LDS; convolutions it does not fit run as tiling 1
      // (measured and not built: a 128 x 128 tile with two or three filter tiles in flight and four filter
      // tiles for this one were 4-30 % slower on every 3x3 layer of ResNet-152 at batch 64)
      if (setting != 0 && patch_kernel_fits<MODE>(a)) return launch_cfg3<MODE, 1, 3>(ctx, a, flops);
      tile_cfg = 1;
    }
    // 9 / 10: 256 x 256 on eight wavefronts (128 x 64 each), two LDS tiles in flight, plain / rotated loop: for
    // products with a thousand such tiles or more (measured on 65 536 x 4096 x 4096: 1.13-1.21 PFLOP/s rotated,
    // 1.02 plain, 0.82-0.91 for 128 x 128; four wavefronts of 128 x 128 each: 0.99-1.05, and slower than 128 x 128
    // on every layer of the three models, like this one)
    if (tile_cfg == 9 || tile_cfg == 10) {
      if (setting != 0 && in_c % kStep2 == 0 && a.R * a.S <= 32)
        return tile_cfg == 9 ? launch_cfg2<MODE, 2, 4, 4, 2, 2>(ctx, a, flops) : launch_cfg2<MODE, 2, 4, 4, 2, 2, 1>(ctx, a, flops);
      tile_cfg = 0;
    }
    // 11 - 14: 32-element reduction steps.  11 / 12: 128 x 128 with three / two LDS tiles in flight (48 / 34 KB:
    // three / four workgroups per CU), 13: 128 x 64 and 14: 64 x 64 with three (36 / 24 KB)
    if (tile_cfg >= 11 && tile_cfg <= 14) {
      if (setting != 0 && in_c % kStep2 == 0 && a.R * a.S <= 32) {
        if (tile_cfg == 11) return launch_cfg2<MODE, 2, 2, 2, 2, 3, 0, 32>(ctx, a, flops);
        if (tile_cfg == 12) return launch_cfg2<MODE, 2, 2, 2, 2, 2, 0, 32>(ctx, a, flops);
        if (tile_cfg == 13) return launch_cfg2<MODE, 2, 2, 2, 1, 3, 0, 32>(ctx, a, flops);
        return launch_cfg2<MODE, 2, 2, 1, 1, 3, 0, 32>(ctx, a, flops);
      }
      tile_cfg = tile_cfg <= 12 ? 0 : tile_cfg - 12;
    }
    // 6 / 7: tilings 1 / 2 with two LDS tiles in flight instead of three (48 / 32 KB of LDS: three or four
    // workgroups per CU, which the memory-bound data gradients of the large feature maps prefer)
    if (tile_cfg == 6 || tile_cfg == 7) {
      if (setting != 0 && in_c % kStep2 == 0 && a.R * a.S <= 32)
        return tile_cfg == 6 ? launch_cfg2<MODE, 2, 2, 2, 1, 2>(ctx, a, flops) : launch_cfg2<MODE, 2, 2, 1, 1, 2>(ctx, a, flops);
      tile_cfg -= 5;
    }
    if (setting != 0 && in_c % kStep2 == 0 && a.R * a.S <= 32 && tile_cfg >= 0 && tile_cfg <= 2) {
      if (tile_cfg == 0)
        return setting == 3 ? launch_cfg2<MODE, 2, 2, 2, 2, 3>(ctx, a, flops) : launch_cfg2<MODE, 2, 2, 2, 2, 2>(ctx, a, flops);
      if (tile_cfg == 1)
        return setting == 2 ? launch_cfg2<MODE, 2, 2, 2, 1, 2>(ctx, a, flops) : launch_cfg2<MODE, 2, 2, 2, 1, 3>(ctx, a, flops);
      return setting == 2 ? launch_cfg2<MODE, 2, 2, 1, 1, 2>(ctx, a, flops) : launch_cfg2<MODE, 2, 2, 1, 1, 3>(ctx, a, flops);
    }
  }
  if (tile_cfg == 5) tile_cfg = 1;
  if (tile_cfg == 6 || tile_cfg == 7) tile_cfg -= 5;
  if (tile_cfg == 9 || tile_cfg == 10) tile_cfg = 0;
  if (tile_cfg >= 11 && tile_cfg <= 14) tile_cfg = tile_cfg <= 12 ? 0 : tile_cfg - 12;
  switch (tile_cfg) {
    case 0:
      return launch_cfg<T, MODE, 2, 2, 2, 2>(ctx, a, flops);  // 128 x 128
    case 1:
      return launch_cfg<T, MODE, 2, 2, 2, 1>(ctx, a, flops);  // 128 x 64
    default:
      return launch_cfg<T, MODE, 2, 2, 1, 1>(ctx, a, flops);  // 64 x 64 (2, and 3 = never the direct-to-LDS kernel)
  }
}

// 2 * N*Ho*Wo * K * R*S*C: the same for forward, data gradient and weight gradient;
// zero-padded input channels do no algorithmic work
double conv_flops(const ConvShape& s, int Ho, int Wo) {
  const int c = (s.c_logical > 0 && s.c_logical < s.C) ? s.c_logical : s.C;
  return 2.0 * s.N * Ho * Wo * static_cast<double>(s.K) * s.R * s.S * c;
}

// rows of the workgroup tile of a tiling number (5 = the 3x3 patch kernel, or tiling 1 where it does not fit)
int tile_rows(int tile_cfg) {
  if (tile_cfg == 9 || tile_cfg == 10) return 256;
  if (tile_cfg >= 11 && tile_cfg <= 14) return tile_cfg == 14 ? 64 : 128;
  return (tile_cfg == 5 || tile_cfg == 6) ? 128 : tile_cfg >= 2 ? 64 : 128;
}

int64_t tiles_for(int m, int n, int bm, int bn) {
  return static_cast<int64_t>((m + bm - 1) / bm) * ((n + bn - 1) / bn);
}

// Whether the 256 x 256 tiling (10) is worth asking for: the kernel it needs is at hand (bf16, reduction in whole
// 64-channel steps, few taps) and the product has at least four full rounds of such tiles.
bool wants_huge_tile(int dtype, int gemm_m, int gemm_n, int in_c, int taps) {
  return dtype == kBF16 && in_c % 64 == 0 && taps <= 32 && igemm2_setting() != 0 &&
         tiles_for(gemm_m, gemm_n, 256, 256) >= 1024;
}

// The tiling that runs when `tile_cfg` is asked for: the 256 x 256 tilings exist for the direct-to-LDS kernel only
// and stand for 128 x 128 elsewhere (the statistics' row tiles follow the tiling that runs).
int effective_tile(int tile_cfg, int dtype, int in_c, int taps) {
  if ((tile_cfg == 9 || tile_cfg == 10) && !(dtype == kBF16 && in_c % 64 == 0 && taps <= 32 && igemm2_setting() != 0))
    return 0;
  return tile_cfg;
}

// Enough workgroups to give each of the 256 CUs some, with bigger tiles as
// soon as the problem can afford them.
int pick_tile(int gemm_m, int gemm_n, int splits) {
  if (gemm_n > 64 && tiles_for(gemm_m, gemm_n, 128, 128) * splits >= 384) return 0;
  if (tiles_for(gemm_m, gemm_n, 128, 64) * splits >= 384) return 1;
  return 2;
}

// The heuristic's tiling for a pointwise product with a shallow reduction (at most 256 channels): the same tile
// shape with 32-element reduction steps (half the LDS per workgroup, more workgroups per CU), which measured faster
// on every such layer of the three models (0 -> 12, 1 -> 13, 2 -> 14: same tile rows, so the statistics' row
// tiles do not change).  TCH_IGEMM_K32=0 keeps the 64-element steps.
int shallow_tile(int tile_cfg, int dtype, int in_c, int taps) {
  static const bool on = [] {
    const char* e = getenv("TCH_IGEMM_K32");
    return !(e && atoi(e) == 0);
  }();
  if (on && dtype == kBF16 && taps == 1 && in_c % 64 == 0 && in_c <= 256 && igemm2_setting() != 0 && tile_cfg >= 0 &&
      tile_cfg <= 2)
    return tile_cfg + 12;
  return tile_cfg;
}

int fill_common(IgemmArgs& a, const ConvShape& s, int dtype) {
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "conv: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(s.N > 0 && s.H > 0 && s.W > 0 && s.C > 0 && s.K > 0 && s.R > 0 && s.S > 0, "conv: non-positive dimension");
  TCH_CHECK_ARG(s.stride >= 1 && ilog2_exact(s.stride) >= 0, "conv: stride must be a power of two");
  TCH_CHECK_ARG(s.pad >= 0 && s.pad < s.R && s.pad < s.S, "conv: padding must be smaller than the filter");
  TCH_CHECK_ARG(s.C % E == 0 && s.K % E == 0, "conv: channel counts must be multiples of a 16-byte chunk");
  const int Ho = (s.H + 2 * s.pad - s.R) / s.stride + 1;
  const int Wo = (s.W + 2 * s.pad - s.S) / s.stride + 1;
  TCH_CHECK_ARG(Ho > 0 && Wo > 0, "conv: empty output");
  const int64_t in_elems = static_cast<int64_t>(s.N) * s.H * s.W * s.C;
  const int64_t out_elems = static_cast<int64_t>(s.N) * Ho * Wo * s.K;
  TCH_CHECK_ARG(in_elems < (1ll << 31) && out_elems < (1ll << 31), "conv: tensor exceeds 2^31 elements");
  TCH_CHECK_ARG(in_elems * (16 / E) < (1ll << 31) && out_elems * (16 / E) < (1ll << 31),
                "conv: tensor exceeds the 2 GiB reach of a buffer offset");
  TCH_CHECK_ARG(static_cast<int64_t>(s.K) * s.R * s.S * s.C < (1ll << 31), "conv: filter exceeds 2^31 elements");
  a.N = s.N;
  a.H = s.H;
  a.W = s.W;
  a.C = s.C;
  a.Ho = Ho;
  a.Wo = Wo;
  a.K = s.K;
  a.R = s.R;
  a.S = s.S;
  a.stride = s.stride;
  a.stride_log2 = ilog2_exact(s.stride);
  a.pad = s.pad;
  a.pointwise = (s.R == 1 && s.S == 1 && s.stride == 1 && s.pad == 0) ? 1 : 0;
  a.splits = 1;
  a.out_f32 = 0;
  a.accumulate = 0;
  a.add = nullptr;
  a.mask = nullptr;
  a.bias = nullptr;
  return 0;
}

}  // namespace

void conv_output_hw(const ConvShape& s, int* Ho, int* Wo) {
  *Ho = (s.H + 2 * s.pad - s.R) / s.stride + 1;
  *Wo = (s.W + 2 * s.pad - s.S) / s.stride + 1;
}

namespace {

bool check_finalize(const BnFinalize* f, bool forward) {
  return f->counters && f->gamma && f->out0 && f->out1 && f->coef && (!forward || f->beta) &&
         ((f->running_mean == nullptr) == (f->running_var == nullptr));
}

void bind_finalize(IgemmArgs& a, const BnFinalize* f) {
  a.fin_counters = f->counters;
  a.fin_gamma = f->gamma;
  a.fin_beta = f->beta;
  a.fin_running_mean = f->running_mean;
  a.fin_running_var = f->running_var;
  a.fin_out0 = f->out0;
  a.fin_out1 = f->out1;
  a.fin_coef = f->coef;
  a.fin_momentum = f->momentum;
  a.fin_eps = f->eps;
  a.fin_accumulate = f->accumulate;
}

}  // namespace

int conv2d_fwd(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* w, void* y, const void* add,
               const void* mask, const float* bias, int out_f32, int tile_cfg, float* bn_partial,
               const BnFinalize* finalize, const float* scale, int relu_out, long long* bn_acc, int bn_acc_copies) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(!((scale || relu_out) && (bn_partial || bn_acc)), "conv2d_fwd: statistics are taken of the plain convolution output");
  TCH_CHECK_ARG(!(bn_acc && (bn_partial || finalize || out_f32)),
                "conv2d_fwd: accumulated statistics replace the per-tile ones and are taken of outputs stored in the compute type");
  TCH_CHECK_ARG(!bn_acc || (bn_acc_copies >= 1 && (bn_acc_copies & (bn_acc_copies - 1)) == 0),
                "conv2d_fwd: the number of accumulator copies must be a power of two");
  a.stat_acc = bn_acc;
  a.stat_acc_copies = bn_acc_copies;
  a.scale = scale;
  a.relu_out = relu_out ? 1 : 0;
  TCH_CHECK_ARG(x && w && y, "conv2d_fwd: null tensor");
  TCH_CHECK_ARG(!(bn_partial && out_f32), "conv2d_fwd: statistics are taken of outputs stored in the compute type");
  TCH_CHECK_ARG(!finalize || (bn_partial && check_finalize(finalize, true)), "conv2d_fwd: incomplete BatchNorm finalize operands");
  a.stats = bn_partial;
  const int eb = dtype == kBF16 ? 2 : 4;
  a.a_src = x;
  a.b_src = w;
  a.a_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * s.H * s.W * s.C * eb);
  a.b_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.K) * s.R * s.S * s.C * eb);
  a.out = y;
  a.add = add;
  a.mask = mask;
  a.bias = bias;
  a.out_f32 = out_f32;
  a.gemm_m = s.N * a.Ho * a.Wo;
  a.gemm_n = s.K;
  a.gemm_k = s.R * s.S * s.C;
  a.k_per_split = (a.gemm_k + 31) / 32 * 32;
  a.div_plane = FastDiv(a.Ho * a.Wo);
  a.div_width = FastDiv(a.Wo);
  if (tile_cfg < 0) {
    tile_cfg = shallow_tile(pick_tile(a.gemm_m, a.gemm_n, 1), dtype, s.C, s.R * s.S);
    // statistics are sized by the caller for the heuristic's row tiles: leave those launches alone
    if (!bn_partial && !bn_acc && wants_huge_tile(dtype, a.gemm_m, a.gemm_n, s.C, s.R * s.S)) tile_cfg = 10;
  }
  tile_cfg = effective_tile(tile_cfg, dtype, s.C, s.R * s.S);
  const int row_tiles = (a.gemm_m + tile_rows(tile_cfg) - 1) / tile_rows(tile_cfg);
  const bool in_kernel = finalize && row_tiles <= kBnFinalizeInKernelTiles;
  if (in_kernel) bind_finalize(a, finalize);
  int rc = dtype == kBF16 ? launch_mode<bf16, kFwd>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                          : launch_mode<float, kFwd>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
  if (rc || !finalize || in_kernel) return rc;
  return bn_fwd_finalize(ctx, bn_partial, row_tiles, s.K, a.gemm_m, finalize->gamma, finalize->beta,
                         finalize->running_mean, finalize->running_var, finalize->out0, finalize->out1, finalize->coef,
                         finalize->momentum, finalize->eps);
}

int conv2d_fwd_stat_rows(const ConvShape& s, int dtype, int tile_cfg) {
  int Ho, Wo;
  conv_output_hw(s, &Ho, &Wo);
  const int gemm_m = s.N * Ho * Wo;
  if (tile_cfg < 0) tile_cfg = pick_tile(gemm_m, s.K, 1);
  tile_cfg = effective_tile(tile_cfg, dtype, s.C, s.R * s.S);
  const int bm = tile_rows(tile_cfg);
  return (gemm_m + bm - 1) / bm;
}

int conv2d_dgrad_stat_rows(const ConvShape& s, int dtype, int tile_cfg) {
  const int gemm_m = s.N * s.H * s.W;
  if (tile_cfg < 0) tile_cfg = pick_tile(gemm_m, s.C, 1);
  tile_cfg = effective_tile(tile_cfg, dtype, s.K, s.R * s.S);
  const int bm = tile_rows(tile_cfg);
  return (gemm_m + bm - 1) / bm;
}

int conv2d_dgrad(Context* ctx, int dtype, const ConvShape& s, const void* dy, const void* wt, void* dx,
                 const void* add, const void* mask, int tile_cfg, const BnBwdSums* bn, int add_stride) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(dy && wt && dx, "conv2d_dgrad: null tensor");
  TCH_CHECK_ARG(add_stride == 1 || add_stride == 2, "conv2d_dgrad: the addend's grid is the output's or every second pixel of it");
  a.add_sub = (add && add_stride == 2) ? 1 : 0;
  if (bn) {
    TCH_CHECK_ARG(bn->x && bn->mean && bn->invstd && ((bn->partial != nullptr) != (bn->acc != nullptr)),
                  "conv2d_dgrad: incomplete BatchNorm operands");
    TCH_CHECK_ARG(!bn->finalize || (bn->partial && check_finalize(bn->finalize, false)),
                  "conv2d_dgrad: incomplete BatchNorm finalize operands");
    TCH_CHECK_ARG(!bn->acc || (bn->acc_copies >= 1 && (bn->acc_copies & (bn->acc_copies - 1)) == 0),
                  "conv2d_dgrad: the number of accumulator copies must be a power of two");
    a.stats = bn->partial;
    a.stat_acc = bn->acc;
    a.stat_acc_copies = bn->acc_copies;
    a.bn_mask = bn->mask;
    a.bn_x = bn->x;
    a.bn_mean = bn->mean;
    a.bn_invstd = bn->invstd;
  }
  const int eb = dtype == kBF16 ? 2 : 4;
  a.a_src = dy;
  a.b_src = wt;
  a.a_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * a.Ho * a.Wo * s.K * eb);
  a.b_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.K) * s.R * s.S * s.C * eb);
  a.out = dx;
  a.add = add;
  a.mask = mask;
  a.gemm_m = s.N * s.H * s.W;
  a.gemm_n = s.C;
  a.gemm_k = s.R * s.S * s.K;
  a.k_per_split = (a.gemm_k + 31) / 32 * 32;
  // 1x1 stride 1: dy is a dense [pixels][K] matrix in the same pixel order as dx
  a.div_plane = FastDiv(s.H * s.W);
  a.div_width = FastDiv(s.W);
  if (tile_cfg < 0) {
    tile_cfg = shallow_tile(pick_tile(a.gemm_m, a.gemm_n, 1), dtype, s.K, s.R * s.S);
    if (!bn && wants_huge_tile(dtype, a.gemm_m, a.gemm_n, s.K, s.R * s.S)) tile_cfg = 10;
  }
  tile_cfg = effective_tile(tile_cfg, dtype, s.K, s.R * s.S);
  const BnFinalize* finalize = bn ? bn->finalize : nullptr;
  const int row_tiles = (a.gemm_m + tile_rows(tile_cfg) - 1) / tile_rows(tile_cfg);
  const bool in_kernel = finalize && row_tiles <= kBnFinalizeInKernelTiles;
  if (in_kernel) bind_finalize(a, finalize);
  int rc = dtype == kBF16 ? launch_mode<bf16, kDgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                          : launch_mode<float, kDgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
  if (rc || !finalize || in_kernel) return rc;
  return bn_bwd_finalize(ctx, bn->partial, row_tiles, s.C, a.gemm_m, finalize->gamma, bn->mean, bn->invstd,
                         finalize->out0, finalize->out1, finalize->coef, finalize->accumulate);
}

int64_t conv2d_wgrad_workspace_bytes(const ConvShape& s, int dtype, int splits) {
  if (splits <= 1) return 0;
  (void)dtype;
  // partial filters, then partial column sums of dy for callers that also want the bias gradient
  return static_cast<int64_t>(splits) * (static_cast<int64_t>(s.K) * s.R * s.S * s.C + s.K) * 4;
}

int conv2d_wgrad_pick_splits(const ConvShape& s, int dtype) {
  const int BK = dtype == kBF16 ? 32 : 16;
  int Ho, Wo;
  conv_output_hw(s, &Ho, &Wo);
  const int64_t pixels = static_cast<int64_t>(s.N) * Ho * Wo;
  const int gemm_m = s.K, gemm_n = s.R * s.S * s.C;
  int64_t tiles = tiles_for(gemm_m, gemm_n, 128, 128);
  if (tiles < 8) tiles = tiles_for(gemm_m, gemm_n, 64, 64);
  // Workgroups to aim for.  The weight gradients run beside the data-gradient chain on a second stream: a
  // launch that does not fill the chip by itself shares it better, and every split costs a partial filter
  // written and read again, so filters of few tiles over short reductions aim lower than wide or long products.
  static const int target_env = [] {
    const char* e = getenv("TCH_WGRAD_WGS");
    return e && atoi(e) > 0 ? atoi(e) : 0;
  }();
  const int target_wgs = target_env ? target_env : (tiles <= 64 && pixels <= 16384) ? 192 : 384;
  int64_t want = (target_wgs + tiles - 1) / tiles;
  int64_t max_by_k = pixels / (4 * BK);  // at least four reduction steps per split
  if (max_by_k < 1) max_by_k = 1;
  if (want > max_by_k) want = max_by_k;
  if (want > 512) want = 512;
  if (want < 1) want = 1;
  return static_cast<int>(want);
}

int conv2d_wgrad_flush(Context* ctx) {
  auto& tr = ctx->trailing_reduce;
  if (!tr.valid) return 0;
  tr.valid = false;
  return launch(ctx, splitk_reduce_kernel, dim3(tr.blocks), dim3(256), tr.args, "splitk_reduce_kernel", tr.bytes, 1);
}

int conv2d_wgrad(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* dy, float* dw, float* workspace,
                 int splits, int accumulate, int tile_cfg, float* dbias, int trailing) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(x && dy && dw, "conv2d_wgrad: null tensor");
  const int eb = dtype == kBF16 ? 2 : 4;
  TCH_CHECK_ARG(splits >= 1, "conv2d_wgrad: splits must be >= 1");
  TCH_CHECK_ARG(splits == 1 || workspace, "conv2d_wgrad: split reduction needs a workspace");
  const int BK = dtype == kBF16 ? 32 : 16;
  a.a_src = dy;
  a.b_src = x;
  a.a_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * a.Ho * a.Wo * s.K * eb);
  a.b_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * s.H * s.W * s.C * eb);
  a.gemm_m = s.K;
  a.gemm_n = s.R * s.S * s.C;
  a.gemm_k = s.N * a.Ho * a.Wo;
  int per = (a.gemm_k + splits - 1) / splits;
  per = (per + BK - 1) / BK * BK;
  splits = (a.gemm_k + per - 1) / per;  // drop empty tail splits
  a.splits = splits;
  a.k_per_split = per;
  a.accumulate = accumulate;
  a.take_pending = trailing ? 1 : 0;
  a.out = splits > 1 ? static_cast<void*>(workspace) : static_cast<void*>(dw);
  float* dbias_partial = workspace ? workspace + static_cast<int64_t>(splits) * a.gemm_m * a.gemm_n : nullptr;
  a.dbias = !dbias ? nullptr : splits > 1 ? dbias_partial : dbias;
  a.div_plane = FastDiv(a.Ho * a.Wo);
  a.div_width = FastDiv(a.Wo);
  if (tile_cfg < 0) {
    static const int big_from = [] {
      const char* e = getenv("TCH_WGRAD_BIG_TILE_WGS");
      return e && atoi(e) > 0 ? atoi(e) : 128;
    }();
    tile_cfg = (a.gemm_m >= 128 && a.gemm_n >= 128 && tiles_for(a.gemm_m, a.gemm_n, 128, 128) * splits >= big_from) ? 0 : 2;
  }
  int rc = dtype == kBF16 ? launch_mode<bf16, kWgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                          : launch_mode<float, kWgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
  if (rc) return rc;
  if (splits > 1) {
    ReduceArgs r{workspace, dw, static_cast<int64_t>(a.gemm_m) * a.gemm_n, splits, accumulate, dbias_partial, dbias,
                 dbias ? a.gemm_m : 0, 0u};
    TCH_CHECK_ARG(r.n % 4 == 0, "conv2d_wgrad: filter size must be a multiple of 4");
    r.first_blocks = static_cast<unsigned>((r.n / 4 + 255) / 256);
    const unsigned blocks = r.first_blocks + static_cast<unsigned>((r.n2 + 255) / 256);
    const double red_bytes = 4.0 * r.n * (splits + 1 + (accumulate ? 1 : 0));
    if (trailing) {
      // not launched now: rides the next weight gradient of this context (which must use ANOTHER workspace), or
      // conv2d_wgrad_flush.  An earlier pending reduction was taken along by the launch above.
      auto& tr = ctx->trailing_reduce;
      tr.valid = true;
      tr.args = r;
      tr.blocks = blocks;
      tr.bytes = red_bytes;
      return 0;
    }
    return launch(ctx, splitk_reduce_kernel, dim3(blocks), dim3(256), r, "splitk_reduce_kernel", red_bytes, 1);
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Grouped weight gradients: the weight gradients of several convolutions (a stage of a network, whose dy tensors
// are all at hand once the data-gradient chain has passed) as ONE launch over a table, plus one launch for the
// split reductions that are left.  Together the convolutions fill the chip, so each needs few splits or none:
// long reduction loops, little or nothing written as partial filters, two launches instead of two per layer.
// ---------------------------------------------------------------------------------------------------------------
namespace {

struct GroupLayout {
  int64_t args_off = 0, red_off = 0, map_off = 0, rmap_off = 0, bytes = 0;
  int64_t wgs = 0, reduce_blocks = 0, workspace_floats = 0;
};

int group_tile(int dtype, int n, const ConvShape* shapes, int tile_cfg) {
  if (tile_cfg == 0 || tile_cfg == 2) return tile_cfg;
  for (int i = 0; i < n; ++i)
    if (shapes[i].K < 128 || shapes[i].R * shapes[i].S * shapes[i].C < 128) return 2;
  return 0;
}

int64_t group_pixels(const ConvShape& s) {
  int Ho, Wo;
  conv_output_hw(s, &Ho, &Wo);
  return static_cast<int64_t>(s.N) * Ho * Wo;
}

// what conv2d_wgrad makes of a requested split count: whole reduction steps per split, no empty tail splits
void normalise_split(int64_t pixels, int BK, int want, int* splits, int* per) {
  if (want < 1) want = 1;
  int64_t p = (pixels + want - 1) / want;
  p = (p + BK - 1) / BK * BK;
  *per = static_cast<int>(p);
  *splits = static_cast<int>((pixels + p - 1) / p);
}

GroupLayout group_layout(int dtype, int n, const ConvShape* shapes, const int* splits, int tile) {
  const int BK = dtype == kBF16 ? 32 : 16;
  const int bm = tile == 0 ? 128 : 64;
  GroupLayout L;
  for (int i = 0; i < n; ++i) {
    const ConvShape& s = shapes[i];
    int sp, per;
    normalise_split(group_pixels(s), BK, splits[i], &sp, &per);
    const int64_t filt = static_cast<int64_t>(s.K) * s.R * s.S * s.C;
    L.wgs += tiles_for(s.K, s.R * s.S * s.C, bm, bm) * sp;
    if (sp > 1) {
      L.workspace_floats += sp * (filt + s.K);
      L.reduce_blocks += (filt / 4 + 255) / 256 + (s.K + 255) / 256;
    }
  }
  auto up = [](int64_t v) { return (v + 255) / 256 * 256; };
  L.args_off = 0;
  L.red_off = up(static_cast<int64_t>(n) * sizeof(IgemmArgs));
  L.map_off = L.red_off + up(static_cast<int64_t>(n) * sizeof(ReduceArgs));
  L.rmap_off = L.map_off + up(L.wgs * static_cast<int64_t>(sizeof(uint2)));
  L.bytes = L.rmap_off + up(L.reduce_blocks * static_cast<int64_t>(sizeof(uint2)));
  return L;
}

}  // namespace

int conv2d_wgrad_group_plan(int dtype, int n, const ConvShape* shapes, int target_wgs, int tile_cfg, int* splits,
                            int64_t* table_bytes, int64_t* workspace_bytes) {
  TCH_CHECK_ARG(n > 0 && shapes && splits, "conv2d_wgrad_group_plan: empty group");
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "conv2d_wgrad_group_plan: dtype must be f32(0) or bf16(1)");
  const int BK = dtype == kBF16 ? 32 : 16;
  const int tile = group_tile(dtype, n, shapes, tile_cfg);
  const int bm = tile == 0 ? 128 : 64;
  if (target_wgs <= 0) target_wgs = 1024;
  constexpr int64_t kMinSteps = 16;   // a split is at least this many reduction steps long
  std::vector<int64_t> steps(n), tiles(n);
  int64_t longest = 1;
  for (int i = 0; i < n; ++i) {
    const ConvShape& s = shapes[i];
    TCH_CHECK_ARG(s.N > 0 && s.H > 0 && s.W > 0 && s.C > 0 && s.K > 0 && s.R > 0 && s.S > 0, "conv: non-positive dimension");
    steps[i] = (group_pixels(s) + BK - 1) / BK;
    tiles[i] = tiles_for(s.K, s.R * s.S * s.C, bm, bm);
    longest = std::max(longest, steps[i]);
  }
  // Every workgroup runs about `len` reduction steps: the largest `len` that still yields target_wgs workgroups
  // (none if the unsplit group already has that many).
  auto wgs_at = [&](int64_t len) {
    int64_t w = 0;
    for (int i = 0; i < n; ++i) w += tiles[i] * ((steps[i] + len - 1) / len);
    return w;
  };
  int64_t len = longest;
  if (wgs_at(len) < target_wgs) {
    int64_t lo = kMinSteps, hi = longest;   // wgs_at is non-increasing in len
    while (lo < hi) {
      const int64_t mid = (lo + hi + 1) / 2;
      if (wgs_at(mid) >= target_wgs) lo = mid; else hi = mid - 1;
    }
    len = lo;
  }
  for (int i = 0; i < n; ++i) {
    int sp, per;
    normalise_split(group_pixels(shapes[i]), BK, static_cast<int>(std::min<int64_t>((steps[i] + len - 1) / len, 512)), &sp, &per);
    splits[i] = sp;
  }
  const GroupLayout L = group_layout(dtype, n, shapes, splits, tile);
  if (table_bytes) *table_bytes = L.bytes;
  if (workspace_bytes) *workspace_bytes = std::max<int64_t>(L.workspace_floats * 4, 4);
  return tile;
}

int conv2d_wgrad_group(Context* ctx, int dtype, int n, const WgradGroupItem* items, int tile_cfg, int accumulate,
                       float* workspace, void* table, int max_wgs) {
  TCH_CHECK_ARG(n > 0 && items && table, "conv2d_wgrad_group: empty group or no table");
  const int eb = dtype == kBF16 ? 2 : 4;
  const int BK = dtype == kBF16 ? 32 : 16;
  std::vector<ConvShape> shapes(n);
  std::vector<int> splits(n);
  for (int i = 0; i < n; ++i) {
    shapes[i] = items[i].shape;
    splits[i] = items[i].splits;
  }
  const int tile = group_tile(dtype, n, shapes.data(), tile_cfg);
  const int bm = tile == 0 ? 128 : 64;
  const GroupLayout L = group_layout(dtype, n, shapes.data(), splits.data(), tile);
  TCH_CHECK_ARG(L.workspace_floats == 0 || workspace, "conv2d_wgrad_group: split reductions need a workspace");
  TCH_CHECK_ARG(L.wgs > 0 && L.wgs <= 0x7fffffff, "conv2d_wgrad_group: grid out of range");

  std::vector<unsigned char> host(static_cast<size_t>(L.bytes), 0);
  IgemmArgs* args = reinterpret_cast<IgemmArgs*>(host.data() + L.args_off);
  ReduceArgs* reds = reinterpret_cast<ReduceArgs*>(host.data() + L.red_off);
  uint2* map = reinterpret_cast<uint2*>(host.data() + L.map_off);
  uint2* rmap = reinterpret_cast<uint2*>(host.data() + L.rmap_off);
  double flops = 0.0, bytes = 0.0, red_bytes = 0.0;
  int64_t ws_off = 0;
  int n_red = 0;
  std::vector<int> order(n);
  for (int i = 0; i < n; ++i) order[i] = i;
  for (int i = 0; i < n; ++i) {
    IgemmArgs& a = args[i];
    const WgradGroupItem& it = items[i];
    if (int rc = fill_common(a, it.shape, dtype)) return rc;
    TCH_CHECK_ARG(it.x && it.dy && it.dw, "conv2d_wgrad_group: null tensor");
    const ConvShape& s = it.shape;
    a.a_src = it.dy;
    a.b_src = it.x;
    a.a_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * a.Ho * a.Wo * s.K * eb);
    a.b_bytes = static_cast<uint32_t>(static_cast<int64_t>(s.N) * s.H * s.W * s.C * eb);
    a.gemm_m = s.K;
    a.gemm_n = s.R * s.S * s.C;
    a.gemm_k = s.N * a.Ho * a.Wo;
    normalise_split(a.gemm_k, BK, it.splits, &a.splits, &a.k_per_split);
    a.accumulate = accumulate;
    a.tiles_m = (a.gemm_m + bm - 1) / bm;
    a.tiles_n = (a.gemm_n + bm - 1) / bm;
    a.div_plane = FastDiv(a.Ho * a.Wo);
    a.div_width = FastDiv(a.Wo);
    const int64_t filt = static_cast<int64_t>(a.gemm_m) * a.gemm_n;
    if (a.splits > 1) {
      float* part = workspace + ws_off;
      float* bias_part = part + a.splits * filt;
      ws_off += a.splits * (filt + a.gemm_m);
      a.out = part;
      a.dbias = it.dbias ? bias_part : nullptr;
      TCH_CHECK_ARG(filt % 4 == 0, "conv2d_wgrad_group: filter size must be a multiple of 4");
      ReduceArgs& r = reds[n_red];
      r = ReduceArgs{part, it.dw, filt, a.splits, accumulate, bias_part, it.dbias, it.dbias ? a.gemm_m : 0, 0u};
      r.first_blocks = static_cast<unsigned>((filt / 4 + 255) / 256);
      red_bytes += 4.0 * filt * (a.splits + 1 + (accumulate ? 1 : 0));
      ++n_red;
    } else {
      a.out = it.dw;
      a.dbias = it.dbias;
    }
    flops += conv_flops(s, a.Ho, a.Wo);
    bytes += conv_bytes<kWgrad>(a, eb);
  }
  // long workgroups first: what is left for the tail of the launch is short
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return args[x].k_per_split > args[y].k_per_split; });
  int64_t w = 0;
  for (int oi = 0; oi < n; ++oi) {
    const int i = order[oi];
    const int64_t cnt = static_cast<int64_t>(args[i].tiles_m) * args[i].tiles_n * args[i].splits;
    for (int64_t j = 0; j < cnt; ++j) map[w++] = make_uint2(static_cast<unsigned>(i), static_cast<unsigned>(j));
  }
  TCH_CHECK_ARG(w == L.wgs, "conv2d_wgrad_group: workgroup count does not match the layout");
  int64_t rb = 0;
  for (int i = 0; i < n_red; ++i) {
    const unsigned cnt = reds[i].first_blocks + static_cast<unsigned>((reds[i].n2 + 255) / 256);
    for (unsigned j = 0; j < cnt; ++j) rmap[rb++] = make_uint2(static_cast<unsigned>(i), j);
  }
  TCH_CHECK_ARG(rb <= L.reduce_blocks, "conv2d_wgrad_group: reduction blocks do not match the layout");
  // The table is written once, here; the launches (recorded or not) read it whenever they run.
  hipError_t e = hipMemcpy(table, host.data(), host.size(), hipMemcpyHostToDevice);
  TCH_CHECK_ARG(e == hipSuccess, std::string("conv2d_wgrad_group: table upload: ") + hipGetErrorString(e));

  unsigned char* dev = static_cast<unsigned char*>(table);
  WgradGroupArgs g{reinterpret_cast<const IgemmArgs*>(dev + L.args_off), reinterpret_cast<const uint2*>(dev + L.map_off),
                   static_cast<uint32_t>(L.wgs)};
  const dim3 grid(static_cast<unsigned>(max_wgs > 0 && max_wgs < L.wgs ? max_wgs : L.wgs)), block(256);
  static const std::string names[2][2] = {{"wgrad_group_kernel<f32,128x128>", "wgrad_group_kernel<f32,64x64>"},
                                          {"wgrad_group_kernel<bf16,128x128>", "wgrad_group_kernel<bf16,64x64>"}};
  const char* name = names[dtype == kBF16 ? 1 : 0][tile == 0 ? 0 : 1].c_str();
  int rc;
  if (dtype == kBF16)
    rc = tile == 0 ? launch(ctx, wgrad_group_kernel<bf16, 2, 2, 2, 2>, grid, block, g, name, flops, 0, bytes)
                   : launch(ctx, wgrad_group_kernel<bf16, 2, 2, 1, 1>, grid, block, g, name, flops, 0, bytes);
  else
    rc = tile == 0 ? launch(ctx, wgrad_group_kernel<float, 2, 2, 2, 2>, grid, block, g, name, flops, 0, bytes)
                   : launch(ctx, wgrad_group_kernel<float, 2, 2, 1, 1>, grid, block, g, name, flops, 0, bytes);
  if (rc) return rc;
  if (rb > 0) {
    ReduceGroupArgs rg{reinterpret_cast<const ReduceArgs*>(dev + L.red_off), reinterpret_cast<const uint2*>(dev + L.rmap_off)};
    return launch(ctx, splitk_reduce_group_kernel, dim3(static_cast<unsigned>(rb)), dim3(256), rg,
                  "splitk_reduce_group_kernel", red_bytes, 1);
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Weight gradient for callers that cannot allocate: the split-K partials go to a buffer that is part of the
// library's own device image, so that no workspace is passed in and none is made.
// ---------------------------------------------------------------------------------------------------------------
}  // namespace tch

// 64 MiB of fp32 partials per GPU, held from the moment the code object is loaded until the process ends.
// Host code never touches this name: it is a host-side stand-in for a device symbol.  The device address comes
// from hipGetSymbolAddress, once per device, and that pointer is what kernels and copies get.
static constexpr int64_t kStaticScratchFloats = 16ll << 20;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

namespace tch {

namespace {
constexpr int kScratchDevices = 16;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kScratchDevices] = {};
// who used the buffer last on each device: a call on another stream waits for that call's reduction first
hipEvent_t g_scratch_done[kScratchDevices] = {};
hipStream_t g_scratch_stream[kScratchDevices] = {};
bool g_scratch_used[kScratchDevices] = {};

// The device address of `scratch` on the current device (every GPU holds its own copy at its own address).
int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  TCH_CHECK_ARG(e == hipSuccess && dev >= 0 && dev < kScratchDevices,
                std::string("conv2d_wgrad_static: hipGetDevice: ") + hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    TCH_CHECK_ARG(e == hipSuccess && ptr, std::string("conv2d_wgrad_static: hipGetSymbolAddress: ") + hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
    // set-up, once per device: the event that orders two streams' use of the buffer
    e = hipEventCreateWithFlags(&g_scratch_done[dev], hipEventDisableTiming);
    TCH_CHECK_ARG(e == hipSuccess, std::string("conv2d_wgrad_static: hipEventCreate: ") + hipGetErrorString(e));
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// Launches that go to a stream right now (not recorded into a program, not held in a launch queue, not captured
// into a graph) are ordered here: the buffer's previous user on ANOTHER stream must have finished its reduction
// before this call's partials overwrite it.  In the other three cases the launches run later, in an order only
// the caller knows: there the caller keeps two users of the buffer apart.
bool orders_itself(Context* ctx, hipStream_t stream) {
  if (ctx->recording || ctx->queue) return false;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) return false;
  return true;
}
}  // namespace

int64_t conv2d_wgrad_static_capacity_bytes() { return kStaticScratchFloats * 4; }

int conv2d_wgrad_static(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* dy, float* dw, int splits,
                        int accumulate, int tile_cfg) {
  const int64_t cap = conv2d_wgrad_static_capacity_bytes();
  const int64_t per_split = conv2d_wgrad_workspace_bytes(s, dtype, 2) / 2;
  TCH_CHECK_ARG(per_split > 0, "conv2d_wgrad_static: empty filter");
  if (splits <= 0) {
    // the library's own choice, lowered to what the buffer holds (one split needs no partials at all)
    splits = conv2d_wgrad_pick_splits(s, dtype);
    if (splits > cap / per_split) splits = static_cast<int>(cap / per_split);
    if (splits < 2) splits = 1;
  } else if (splits > 1 && conv2d_wgrad_workspace_bytes(s, dtype, splits) > cap) {
    TCH_CHECK_ARG(false, "conv2d_wgrad_static: " + std::to_string(splits) + " splits of this filter need " +
                             std::to_string(conv2d_wgrad_workspace_bytes(s, dtype, splits)) +
                             " bytes of split-K partials, the static buffer holds " + std::to_string(cap));
  }
  float* ptr = nullptr;
  if (splits > 1)
    if (int rc = static_scratch(&ptr)) return rc;
  // Every partial element the reduction reads is written by the split kernels of the same call first, so
  // what an earlier call left in the buffer never shows; two calls that overlap on one GPU would race on it.
  if (splits <= 1) return conv2d_wgrad(ctx, dtype, s, x, dy, dw, ptr, splits, accumulate, tile_cfg);
  int dev = 0;
  (void)hipGetDevice(&dev);
  const hipStream_t stream = ctx->main_stream();
  const bool ordered = orders_itself(ctx, stream);
  std::lock_guard<std::mutex> lock(g_scratch_mu);   // two host threads do not interleave their launches either
  if (ordered && g_scratch_used[dev] && g_scratch_stream[dev] != stream)
    (void)hipStreamWaitEvent(stream, g_scratch_done[dev], 0);
  const int rc = conv2d_wgrad(ctx, dtype, s, x, dy, dw, ptr, splits, accumulate, tile_cfg);
  if (ordered && rc == 0 && hipEventRecord(g_scratch_done[dev], stream) == hipSuccess) {
    g_scratch_stream[dev] = stream;
    g_scratch_used[dev] = true;
  }
  return rc;
}

}  // namespace tch
