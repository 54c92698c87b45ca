// Training-mode BatchNorm over NHWC activations viewed as [rows, C], with the
// ReLU and the residual add of a bottleneck block fused into the apply pass.
// HBM-bound: every pass moves 16-byte chunks per lane, channel = fastest dim.
//
// Arithmetic restated from torch.nn.BatchNorm2d as used by torchvision's
// ResNet (reference call site train/resnet152.py:22): batch statistics with
// biased variance for normalisation, unbiased variance into running_var,
// momentum update running = (1-m)*running + m*batch.
//
//   forward : partial (sum, sum of squares) per row block  -> finalize (fp64)
//             -> y = relu(x*scale + shift [+ residual])
//   backward: g = dy * (mask > 0); partial (sum g, sum g*xhat) -> finalize
//             -> dx = gamma*invstd*(g - mean(g) - xhat*mean(g*xhat))
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

struct ColReduceArgs {
  const void* a;     // stats: x        bwd: dy
  const void* mask;  // bwd: tensor whose sign gates dy (may be null)
  const void* x;     // bwd: x
  const float* mean;
  const float* invstd;
  float* partial;  // [row_blocks][C][2]
  int64_t rows;
  int C, cc, ccb, rowlanes;
  int64_t rows_per_block;
};

template <typename T, int BWD>
__global__ __launch_bounds__(256) void col_reduce_kernel(ColReduceArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  __shared__ float red[256 * 2 * E];
  const int tid = threadIdx.x;
  const int tx = tid % p.ccb, ty = tid / p.ccb;
  const int col = blockIdx.x * p.ccb + tx;  // chunk column
  const bool col_ok = col < p.cc;
  float s1[E], s2[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s1[e] = s2[e] = 0.f;
  float mu[E], is[E];
  if (BWD && col_ok) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      mu[e] = p.mean[col * E + e];
      is[e] = p.invstd[col * E + e];
    }
  }
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * p.rows_per_block;
  int64_t r1 = r0 + p.rows_per_block;
  if (r1 > p.rows) r1 = p.rows;
  if (col_ok) {
    for (int64_t r = r0 + ty; r < r1; r += p.rowlanes) {
      const int64_t ci = r * p.cc + col;
      Chunk ca;
      ca.u = static_cast<const uint4*>(p.a)[ci];
      float va[E];
      chunk_to_float<T>(ca, va);
      if (BWD) {
        Chunk cx;
        cx.u = static_cast<const uint4*>(p.x)[ci];
        float vx[E];
        chunk_to_float<T>(cx, vx);
        if (p.mask) {
          Chunk cm;
          cm.u = static_cast<const uint4*>(p.mask)[ci];
          float vm[E];
          chunk_to_float<T>(cm, vm);
#pragma unroll
          for (int e = 0; e < E; ++e)
            if (!(vm[e] > 0.f)) va[e] = 0.f;
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
          s1[e] += va[e];
          s2[e] += va[e] * ((vx[e] - mu[e]) * is[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          s1[e] += va[e];
          s2[e] += va[e] * va[e];
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) {
    red[(tid * 2 * E) + e] = s1[e];
    red[(tid * 2 * E) + E + e] = s2[e];
  }
  __syncthreads();
  if (ty == 0 && col_ok) {
    for (int y = 1; y < p.rowlanes; ++y) {
      const float* o = red + ((y * p.ccb + tx) * 2 * E);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        s1[e] += o[e];
        s2[e] += o[E + e];
      }
    }
    float* dst = p.partial + (static_cast<int64_t>(blockIdx.y) * p.C + col * E) * 2;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      dst[2 * e] = s1[e];
      dst[2 * e + 1] = s2[e];
    }
  }
}

struct FwdFinalizeArgs {
  const float* partial;
  int row_blocks, C;
  int64_t rows;
  const float* gamma;
  const float* beta;
  float* running_mean;
  float* running_var;
  float* save_mean;
  float* save_invstd;
  float* scale;
  float* shift;
  float momentum, eps;
};

// Sum the per-row-block partials of one channel: 8 channels x 128 lanes per workgroup (thread = lane * 8 +
// channel, so the 8 channels of a row block are one 64-byte piece).  What this costs is its count of
// dependent round trips to L2, so every lane requests 16 row blocks at once: up to 2048 row blocks are one
// trip.  The lanes add up in fp64 in a fixed order: own values, the 8 lanes of a wavefront by exchange, the
// 16 wavefronts through LDS.
constexpr int kFinalizeThreads = 1024;
__device__ inline bool finalize_sums(const float* partial, int row_blocks, int C, int c, int lane, double* s_out,
                                     double* q_out) {
  constexpr int LANES = kFinalizeThreads / 8, WAVES = kFinalizeThreads / 64;
  __shared__ double red[WAVES][8][2];
  double s = 0.0, q = 0.0;
  if (c < C) {
    constexpr int U = 16;
    for (int b = lane; b < row_blocks; b += U * LANES) {
      float2 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int bb = b + u * LANES;   // past the end: the last row block again, counted as zero
        v[u] = *reinterpret_cast<const float2*>(partial + (static_cast<int64_t>(bb < row_blocks ? bb : row_blocks - 1) * C + c) * 2);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (b + u * LANES >= row_blocks) v[u] = make_float2(0.f, 0.f);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        s += v[u].x;
        q += v[u].y;
      }
    }
  }
#pragma unroll
  for (int off = 8; off < 64; off <<= 1) {
    s += __shfl_xor(s, off, 64);
    q += __shfl_xor(q, off, 64);
  }
  const int cl = threadIdx.x & 7, wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) < 8) {
    red[wave][cl][0] = s;
    red[wave][cl][1] = q;
  }
  __syncthreads();
  s = q = 0.0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    s += red[w][cl][0];
    q += red[w][cl][1];
  }
  *s_out = s;
  *q_out = q;
  return lane == 0 && c < C;
}

__global__ __launch_bounds__(kFinalizeThreads) void bn_fwd_finalize_kernel(FwdFinalizeArgs p) {
  const int c = blockIdx.x * 8 + (threadIdx.x & 7);
  double s, q;
  if (!finalize_sums(p.partial, p.row_blocks, p.C, c, threadIdx.x >> 3, &s, &q)) return;
  const double n = static_cast<double>(p.rows);
  const double mean = s / n;
  double var = q / n - mean * mean;
  if (var < 0.0) var = 0.0;
  const float invstd = 1.0f / sqrtf(static_cast<float>(var) + p.eps);
  p.save_mean[c] = static_cast<float>(mean);
  p.save_invstd[c] = invstd;
  if (p.running_mean) {
    const double unbiased = p.rows > 1 ? var * n / (n - 1.0) : var;
    p.running_mean[c] = (1.f - p.momentum) * p.running_mean[c] + p.momentum * static_cast<float>(mean);
    p.running_var[c] = (1.f - p.momentum) * p.running_var[c] + p.momentum * static_cast<float>(unbiased);
  }
  const float sc = p.gamma[c] * invstd;
  p.scale[c] = sc;
  p.shift[c] = p.beta[c] - static_cast<float>(mean) * sc;
}

struct BwdFinalizeArgs {
  const float* partial;
  int row_blocks, C;
  int64_t rows;
  const float* gamma;
  const float* mean;
  const float* invstd;
  float* dgamma;
  float* dbeta;
  float* coef;  // [3][C]: dx = coef0*g + coef1*x + coef2
  int accumulate;
};

__global__ __launch_bounds__(kFinalizeThreads) void bn_bwd_finalize_kernel(BwdFinalizeArgs p) {
  const int c = blockIdx.x * 8 + (threadIdx.x & 7);
  double s1, s2;
  if (!finalize_sums(p.partial, p.row_blocks, p.C, c, threadIdx.x >> 3, &s1, &s2)) return;
  const float db = static_cast<float>(s1), dg = static_cast<float>(s2);
  p.dbeta[c] = p.accumulate ? p.dbeta[c] + db : db;
  p.dgamma[c] = p.accumulate ? p.dgamma[c] + dg : dg;
  const double n = static_cast<double>(p.rows);
  const double scale = static_cast<double>(p.gamma[c]) * p.invstd[c];
  const double cb = -scale * p.invstd[c] * (s2 / n);
  const double c0 = -scale * (s1 / n) - cb * p.mean[c];
  p.coef[c] = static_cast<float>(scale);
  p.coef[p.C + c] = static_cast<float>(cb);
  p.coef[2 * p.C + c] = static_cast<float>(c0);
}

struct ApplyArgs {
  const void* a;     // fwd: x         bwd: dy
  const void* b;     // fwd: residual  bwd: relu mask   (may be null)
  const void* x;     // bwd: x
  void* out;         // fwd: y         bwd: dx
  const float* c0;   // fwd: scale     bwd: coef0
  const float* c1;   // fwd: shift     bwd: coef1
  const float* c2;   //                bwd: coef2
  int64_t chunks;
  FastDiv div_cc;
  int relu;
  int64_t rows;        // bn_apply_cols_kernel: rows of the tensor and rows per workgroup slab
  int rows_per_slab;
  int nt;
};

template <typename T, int BWD>
__global__ __launch_bounds__(256) void bn_apply_kernel(ApplyArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < p.chunks; i += stride) {
    // chunk column: i % cc, evaluated on the low 31 bits when i is large
    uint32_t colq, col;
    if (i < 0x7fffffffll) {
      p.div_cc.divmod(static_cast<uint32_t>(i), colq, col);
    } else {
      col = static_cast<uint32_t>(i % p.div_cc.d);
    }
    const int ch = col * E;
    Chunk ca;
    ca.u = static_cast<const uint4*>(p.a)[i];
    float va[E], vo[E];
    chunk_to_float<T>(ca, va);
    if (BWD) {
      Chunk cx;
      cx.u = static_cast<const uint4*>(p.x)[i];
      float vx[E];
      chunk_to_float<T>(cx, vx);
      if (p.b) {
        Chunk cm;
        cm.u = static_cast<const uint4*>(p.b)[i];
        float vm[E];
        chunk_to_float<T>(cm, vm);
#pragma unroll
        for (int e = 0; e < E; ++e)
          if (!(vm[e] > 0.f)) va[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < E; ++e) vo[e] = p.c0[ch + e] * va[e] + p.c1[ch + e] * vx[e] + p.c2[ch + e];
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e) vo[e] = va[e] * p.c0[ch + e] + p.c1[ch + e];
      if (p.b) {
        Chunk cr;
        cr.u = static_cast<const uint4*>(p.b)[i];
        float vr[E];
        chunk_to_float<T>(cr, vr);
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] += vr[e];
      }
      if (p.relu) {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = vo[e] > 0.f ? vo[e] : 0.f;
      }
    }
    static_cast<uint4*>(p.out)[i] = float_to_chunk<T>(vo).u;
  }
}

// The same with the coefficients resident: a thread keeps one 16-byte chunk column (its 4 or 8 channels'
// coefficients in registers, loaded once) and walks down the rows of its workgroup's slab, four rows per trip,
// all of them requested before any is used.  bn_apply_kernel fetches 64-96 bytes of coefficients from the cache
// per 16-byte chunk of data; this one none.  CPR chunk columns per workgroup (CPR * 16 contiguous bytes per row).
template <typename T, int BWD, int CPR>
__global__ __launch_bounds__(256) void bn_apply_cols_kernel(ApplyArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int RPP = 256 / CPR;   // rows per pass of the workgroup
  constexpr int U = 4;
  const int tx = threadIdx.x % CPR, ty = threadIdx.x / CPR;
  const int64_t cc = p.div_cc.d;
  const int64_t col_chunk = static_cast<int64_t>(blockIdx.x) * CPR + tx;
  const int ch = static_cast<int>(col_chunk) * E;
  float k0[E], k1[E], k2[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    k0[e] = p.c0[ch + e];
    k1[e] = p.c1[ch + e];
    k2[e] = BWD ? p.c2[ch + e] : 0.f;
  }
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * p.rows_per_slab;
  int64_t r1 = r0 + p.rows_per_slab;
  if (r1 > p.rows) r1 = p.rows;
  for (int64_t r = r0 + ty; r < r1; r += U * RPP) {
    Chunk ca[U], cb[U], cx[U];
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const int64_t row = r + q * RPP;
      ca[q] = cb[q] = cx[q] = zero_chunk();
      if (row < r1) {
        const int64_t i = row * cc + col_chunk;
        if (p.nt) {
          ca[q].u = load_streaming_u4(p.a, i);
          if (BWD) cx[q].u = load_streaming_u4(p.x, i);
          if (p.b) cb[q].u = load_streaming_u4(p.b, i);
        } else {
          ca[q].u = static_cast<const uint4*>(p.a)[i];
          if (BWD) cx[q].u = static_cast<const uint4*>(p.x)[i];
          if (p.b) cb[q].u = static_cast<const uint4*>(p.b)[i];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const int64_t row = r + q * RPP;
      if (row >= r1) continue;
      float va[E], vb[E], vo[E];
      chunk_to_float<T>(ca[q], va);
      chunk_to_float<T>(cb[q], vb);
      if (BWD) {
        float vx[E];
        chunk_to_float<T>(cx[q], vx);
        if (p.b) {
#pragma unroll
          for (int e = 0; e < E; ++e)
            if (!(vb[e] > 0.f)) va[e] = 0.f;
        }
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = k0[e] * va[e] + k1[e] * vx[e] + k2[e];
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = va[e] * k0[e] + k1[e];
        if (p.b) {
#pragma unroll
          for (int e = 0; e < E; ++e) vo[e] += vb[e];
        }
        if (p.relu) {
#pragma unroll
          for (int e = 0; e < E; ++e) vo[e] = vo[e] > 0.f ? vo[e] : 0.f;
        }
      }
      static_cast<uint4*>(p.out)[row * cc + col_chunk] = float_to_chunk<T>(vo).u;
    }
  }
}

// Finalize + apply in ONE launch, for layers whose sums come in few rows (the 14x14 and 7x7 stages, where a
// launch costs more than the work): a workgroup owns 64 channels and a slab of rows; it first sums the
// per-tile partials of its 64 channels itself (every workgroup of a column block repeats that sum, in the
// same fixed order, from L2: row_blocks x 512 bytes), then applies.  The workgroups of slab 0 also write the
// per-channel outputs (saved statistics, running statistics / dgamma, dbeta).
constexpr int kFusedCols = 64;
constexpr int kFusedMaxRowBlocks = 256;

struct FinApplyArgs {
  const float* partial;
  int row_blocks, C;
  int64_t rows;
  const float* gamma;
  const float* beta;      // forward
  float* running_mean;    // forward (may be null)
  float* running_var;
  float* save_mean;       // forward: written   backward: read
  float* save_invstd;
  float* dgamma;          // backward
  float* dbeta;
  float momentum, eps;
  int accumulate;
  const void* a;          // forward: x         backward: g
  const void* b;          // forward: residual (may be null)   backward: x
  void* out;
  int relu;
  int rows_per_slab;
};

template <typename T, int BWD>
__global__ __launch_bounds__(256) void bn_fin_apply_kernel(FinApplyArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int CPR = kFusedCols / E;     // chunks of this workgroup's channels per row
  constexpr int RPP = 256 / CPR;          // rows per pass
  __shared__ double red[8][32][4];
  __shared__ float coef[3][kFusedCols];
  const int tid = threadIdx.x;
  const int c0 = blockIdx.x * kFusedCols;
  {
    const int pr = tid & 31, part = tid >> 5;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    constexpr int U = 16;   // 128 row blocks per round trip
    // uniform base + 32-bit lane offset: one address register per request
    const float* base = p.partial + static_cast<int64_t>(c0) * 2;
    const uint32_t stride = static_cast<uint32_t>(p.C) * 2;   // floats per row block
    for (int b = part; b < p.row_blocks; b += 8 * U) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // every request is made (a row block past the end repeats the last one and counts as zero): a
        // conditional request would be a branch of its own
        const int bb = b + 8 * u;
        const uint32_t off = static_cast<uint32_t>(bb < p.row_blocks ? bb : p.row_blocks - 1) * stride + 4u * pr;
        v[u] = *reinterpret_cast<const float4*>(base + off);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (b + 8 * u >= p.row_blocks) v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // keeps the conversions to fp64 next to their additions (hoisted, they would cost 2 registers per value)
        if (u % 4 == 0) __builtin_amdgcn_sched_barrier(0);
        s0 += v[u].x;
        q0 += v[u].y;
        s1 += v[u].z;
        q1 += v[u].w;
      }
    }
    red[part][pr][0] = s0;
    red[part][pr][1] = q0;
    red[part][pr][2] = s1;
    red[part][pr][3] = q1;
  }
  __syncthreads();
  if (tid < kFusedCols) {
    const int c = c0 + tid;
    double s = 0.0, q = 0.0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      s += red[k][tid >> 1][(tid & 1) * 2];
      q += red[k][tid >> 1][(tid & 1) * 2 + 1];
    }
    const double n = static_cast<double>(p.rows);
    const bool writer = blockIdx.y == 0;
    if (!BWD) {
      const double mean = s / n;
      double var = q / n - mean * mean;
      if (var < 0.0) var = 0.0;
      const float invstd = 1.0f / sqrtf(static_cast<float>(var) + p.eps);
      const float sc = p.gamma[c] * invstd;
      coef[0][tid] = sc;
      coef[1][tid] = p.beta[c] - static_cast<float>(mean) * sc;
      if (writer) {
        p.save_mean[c] = static_cast<float>(mean);
        p.save_invstd[c] = invstd;
        if (p.running_mean) {
          const double unbiased = p.rows > 1 ? var * n / (n - 1.0) : var;
          p.running_mean[c] = (1.f - p.momentum) * p.running_mean[c] + p.momentum * static_cast<float>(mean);
          p.running_var[c] = (1.f - p.momentum) * p.running_var[c] + p.momentum * static_cast<float>(unbiased);
        }
      }
    } else {
      const double invstd = p.save_invstd[c];
      const double scale = static_cast<double>(p.gamma[c]) * invstd;
      const double cb = -scale * invstd * (q / n);
      const double cz = -scale * (s / n) - cb * p.save_mean[c];
      coef[0][tid] = static_cast<float>(scale);
      coef[1][tid] = static_cast<float>(cb);
      coef[2][tid] = static_cast<float>(cz);
      if (writer) {
        const float db = static_cast<float>(s), dg = static_cast<float>(q);
        p.dbeta[c] = p.accumulate ? p.dbeta[c] + db : db;
        p.dgamma[c] = p.accumulate ? p.dgamma[c] + dg : dg;
      }
    }
  }
  __syncthreads();

  const int tx = tid % CPR, ty = tid / CPR;
  float k0[E], k1[E], k2[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    k0[e] = coef[0][tx * E + e];
    k1[e] = coef[1][tx * E + e];
    k2[e] = BWD ? coef[2][tx * E + e] : 0.f;
  }
  const int64_t cc = p.C / E;                    // chunks per full row
  const int64_t col_chunk = c0 / E + tx;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * p.rows_per_slab;
  int64_t r1 = r0 + p.rows_per_slab;
  if (r1 > p.rows) r1 = p.rows;
  const bool has_b = BWD || p.b != nullptr;
  auto finish = [&](int64_t i, const Chunk& ca, const Chunk& cb) {
    float va[E], vb[E], vo[E];
    chunk_to_float<T>(ca, va);
    chunk_to_float<T>(cb, vb);
    if (BWD) {
#pragma unroll
      for (int e = 0; e < E; ++e) vo[e] = k0[e] * va[e] + k1[e] * vb[e] + k2[e];
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e) vo[e] = va[e] * k0[e] + k1[e];
      if (p.b) {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] += vb[e];
      }
      if (p.relu) {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = vo[e] > 0.f ? vo[e] : 0.f;
      }
    }
    static_cast<uint4*>(p.out)[i] = float_to_chunk<T>(vo).u;
  };
  // two rows per trip: both rows' chunks are requested before either is used
  for (int64_t r = r0 + ty; r < r1; r += 2 * RPP) {
    const int64_t i0 = r * cc + col_chunk, i1 = i0 + RPP * cc;
    const bool second = r + RPP < r1;
    Chunk a0, a1, b0 = zero_chunk(), b1 = zero_chunk();
    a0.u = static_cast<const uint4*>(p.a)[i0];
    if (has_b) b0.u = static_cast<const uint4*>(p.b)[i0];
    a1 = a0;
    if (second) {
      a1.u = static_cast<const uint4*>(p.a)[i1];
      if (has_b) b1.u = static_cast<const uint4*>(p.b)[i1];
    }
    finish(i0, a0, b0);
    if (second) finish(i1, a1, b1);
  }
}

// Coefficients from exact accumulators AND apply in one launch, for any number of rows: the convolution next to
// the BatchNorm added its per-tile sums to one pair of accumulators per channel (acc_add), so there are no
// per-tile partials to add up and no finalize launch.  A workgroup owns CPR chunk columns (CPR * E channels, at
// most 256: one thread per channel turns the two totals into the channel's coefficients, through LDS) and a slab
// of rows, which it walks like bn_apply_cols_kernel: a thread keeps one chunk column, four rows per trip.  The
// workgroups of slab 0 also write the per-channel outputs (saved statistics, running statistics / dgamma, dbeta).
struct AccApplyArgs {
  const long long* acc;   // [copies][4][C]: forward sum x, sum x^2; backward sum g, sum g * xhat
  int acc_copies;
  int C;
  int64_t rows;
  const float* gamma;
  const float* beta;      // forward
  float* running_mean;    // forward (may be null)
  float* running_var;
  float* save_mean;       // forward: written   backward: read
  float* save_invstd;
  float* dgamma;          // backward
  float* dbeta;
  float momentum, eps;
  int accumulate;
  const void* a;          // forward: x         backward: g
  const void* b;          // forward: residual (may be null)   backward: x
  void* out;
  int relu;
  int rows_per_slab;
  int nt;                 // stream the inputs past the caches
};

template <typename T, int BWD, int CPR>
__global__ __launch_bounds__(256) void bn_acc_apply_kernel(AccApplyArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int COLS = CPR * E;
  static_assert(COLS <= 256, "one thread per channel of the workgroup");
  constexpr int RPP = 256 / CPR;   // rows per pass of the workgroup
  constexpr int U = 4;
  __shared__ float coef[3][COLS];
  const int tid = threadIdx.x;
  const int c0 = blockIdx.x * COLS;
  if (tid < COLS) {
    const int c = c0 + tid;
    double s, q;
    acc_totals(p.acc, p.C, p.acc_copies, c, &s, &q);
    const double n = static_cast<double>(p.rows);
    const bool writer = blockIdx.y == 0;
    if (!BWD) {
      const double mean = s / n;
      double var = q / n - mean * mean;
      if (var < 0.0) var = 0.0;
      const float invstd = 1.0f / sqrtf(static_cast<float>(var) + p.eps);
      const float sc = p.gamma[c] * invstd;
      coef[0][tid] = sc;
      coef[1][tid] = p.beta[c] - static_cast<float>(mean) * sc;
      if (writer) {
        p.save_mean[c] = static_cast<float>(mean);
        p.save_invstd[c] = invstd;
        if (p.running_mean) {
          const double unbiased = p.rows > 1 ? var * n / (n - 1.0) : var;
          p.running_mean[c] = (1.f - p.momentum) * p.running_mean[c] + p.momentum * static_cast<float>(mean);
          p.running_var[c] = (1.f - p.momentum) * p.running_var[c] + p.momentum * static_cast<float>(unbiased);
        }
      }
    } else {
      const double invstd = p.save_invstd[c];
      const double scale = static_cast<double>(p.gamma[c]) * invstd;
      const double cb = -scale * invstd * (q / n);
      const double cz = -scale * (s / n) - cb * p.save_mean[c];
      coef[0][tid] = static_cast<float>(scale);
      coef[1][tid] = static_cast<float>(cb);
      coef[2][tid] = static_cast<float>(cz);
      if (writer) {
        const float db = static_cast<float>(s), dg = static_cast<float>(q);
        p.dbeta[c] = p.accumulate ? p.dbeta[c] + db : db;
        p.dgamma[c] = p.accumulate ? p.dgamma[c] + dg : dg;
      }
    }
  }
  __syncthreads();

  const int tx = tid % CPR, ty = tid / CPR;
  float k0[E], k1[E], k2[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    k0[e] = coef[0][tx * E + e];
    k1[e] = coef[1][tx * E + e];
    k2[e] = BWD ? coef[2][tx * E + e] : 0.f;
  }
  const int64_t cc = p.C / E;
  const int64_t col_chunk = static_cast<int64_t>(blockIdx.x) * CPR + tx;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * p.rows_per_slab;
  int64_t r1 = r0 + p.rows_per_slab;
  if (r1 > p.rows) r1 = p.rows;
  const bool has_b = BWD || p.b != nullptr;
  for (int64_t r = r0 + ty; r < r1; r += U * RPP) {
    Chunk ca[U], cb[U];
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const int64_t row = r + q * RPP;
      ca[q] = cb[q] = zero_chunk();
      if (row < r1) {
        const int64_t i = row * cc + col_chunk;
        if (p.nt) {
          ca[q].u = load_streaming_u4(p.a, i);
          if (has_b) cb[q].u = load_streaming_u4(p.b, i);
        } else {
          ca[q].u = static_cast<const uint4*>(p.a)[i];
          if (has_b) cb[q].u = static_cast<const uint4*>(p.b)[i];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const int64_t row = r + q * RPP;
      if (row >= r1) continue;
      float va[E], vb[E], vo[E];
      chunk_to_float<T>(ca[q], va);
      chunk_to_float<T>(cb[q], vb);
      if (BWD) {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = k0[e] * va[e] + k1[e] * vb[e] + k2[e];
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) vo[e] = va[e] * k0[e] + k1[e];
        if (p.b) {
#pragma unroll
          for (int e = 0; e < E; ++e) vo[e] += vb[e];
        }
        if (p.relu) {
#pragma unroll
          for (int e = 0; e < E; ++e) vo[e] = vo[e] > 0.f ? vo[e] : 0.f;
        }
      }
      static_cast<uint4*>(p.out)[row * cc + col_chunk] = float_to_chunk<T>(vo).u;
    }
  }
}

// Workgroups to aim for: a small tensor (the 14x14 and 7x7 stages) wants few, since every workgroup repeats the
// coefficient prologue; a large one wants many short ones (TCH_BN_ACC_WGS / TCH_BN_ACC_WGS_LARGE).
template <typename T, int BWD, int CPR>
int launch_acc_apply(Context* ctx, AccApplyArgs& a, const char* name, double bytes) {
  static const int target_small = [] {
    const char* e = getenv("TCH_BN_ACC_WGS");
    return e && atoi(e) > 0 ? atoi(e) : 512;
  }();
  static const int target_large = [] {
    const char* e = getenv("TCH_BN_ACC_WGS_LARGE");
    return e && atoi(e) > 0 ? atoi(e) : 4096;
  }();
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int trip = 4 * (256 / CPR);
  const int64_t col_blocks = a.C / (CPR * E);
  const double tensor_mb = static_cast<double>(a.rows) * a.C * sizeof(T) / 1e6;
  const int target = tensor_mb > 40.0 ? target_large : target_small;
  int64_t slabs = target / col_blocks;
  if (slabs < 1) slabs = 1;
  int64_t rps = (a.rows + slabs - 1) / slabs;
  rps = (rps + trip - 1) / trip * trip;
  a.rows_per_slab = static_cast<int>(rps);
  static const int nt = [] {
    const char* e = getenv("TCH_BN_APPLY_NT");
    return e ? atoi(e) : 1;
  }();
  a.nt = (nt && tensor_mb > 40.0) ? 1 : 0;   // small tensors were just written and sit in the caches
  const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>((a.rows + rps - 1) / rps));
  return launch(ctx, bn_acc_apply_kernel<T, BWD, CPR>, grid, dim3(256), a, name, bytes, 1);
}

template <typename T, int BWD>
int launch_acc_apply_t(Context* ctx, AccApplyArgs& a, const char* name, double bytes) {
  constexpr int E = Elem<T>::kPerChunk;
  const int cc = a.C / E;
  if (cc % 32 == 0) return launch_acc_apply<T, BWD, 32>(ctx, a, name, bytes);
  if (cc % 16 == 0) return launch_acc_apply<T, BWD, 16>(ctx, a, name, bytes);
  return launch_acc_apply<T, BWD, 8>(ctx, a, name, bytes);
}

// rows per slab so that the grid has about 512 workgroups (TCH_BN_FUSED_WGS), at least 32 rows each: alone the
// kernel takes the same time with 512 to 1024, in the step 512 is 0.1 ms faster (every workgroup repeats the
// sum over the partials, and the weight gradients on the other stream want the room)
int fused_rows_per_slab(int64_t rows, int C) {
  const int col_blocks = C / kFusedCols;
  static const int target = [] {
    const char* e = getenv("TCH_BN_FUSED_WGS");
    return e && atoi(e) > 0 ? atoi(e) : 512;
  }();
  int64_t slabs = target / col_blocks;
  if (slabs < 1) slabs = 1;
  int64_t rps = (rows + slabs - 1) / slabs;
  if (rps < 32) rps = 32;
  return static_cast<int>(rps);
}

bool use_fused_finalize() {
  static const bool on = [] {
    const char* e = getenv("TCH_BN_FUSED_FINALIZE");
    return !e || atoi(e) != 0;
  }();
  return on;
}

struct Geometry {
  int cc, ccb, col_blocks, rowlanes, row_blocks;
  int64_t rows_per_block;
};

Geometry geometry(int64_t rows, int C, int dtype) {
  const int E = dtype == kBF16 ? 8 : 4;
  Geometry g;
  g.cc = C / E;
  int ccb = 1;
  while (ccb < g.cc && ccb < 32) ccb <<= 1;
  g.ccb = ccb;
  g.col_blocks = (g.cc + ccb - 1) / ccb;
  g.rowlanes = 256 / ccb;
  int64_t rb = rows / (static_cast<int64_t>(g.rowlanes) * 8);
  int64_t cap = 1024 / g.col_blocks;
  if (cap < 1) cap = 1;
  if (rb > cap) rb = cap;
  if (rb < 1) rb = 1;
  g.rows_per_block = (rows + rb - 1) / rb;
  g.row_blocks = static_cast<int>((rows + g.rows_per_block - 1) / g.rows_per_block);
  return g;
}

unsigned apply_blocks(int64_t chunks) {
  int64_t b = (chunks + 255) / 256;
  if (b > 8192) b = 8192;
  if (b < 1) b = 1;
  return static_cast<unsigned>(b);
}

template <typename T, int BWD, int CPR>
int launch_apply_cols(Context* ctx, ApplyArgs& a, const char* name, double bytes) {
  static const int target = [] {
    const char* e = getenv("TCH_BN_APPLY_WGS");
    return e && atoi(e) > 0 ? atoi(e) : 8192;
  }();
  constexpr int trip = 4 * (256 / CPR);   // rows a workgroup takes per trip
  const int64_t col_blocks = a.div_cc.d / CPR;
  int64_t slabs = target / col_blocks;
  if (slabs < 1) slabs = 1;
  int64_t rps = (a.rows + slabs - 1) / slabs;
  rps = (rps + trip - 1) / trip * trip;
  a.rows_per_slab = static_cast<int>(rps);
  static const int nt = [] {
    const char* e = getenv("TCH_BN_APPLY_NT");
    return e ? atoi(e) : 1;
  }();
  a.nt = nt;
  const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>((a.rows + rps - 1) / rps));
  return launch(ctx, bn_apply_cols_kernel<T, BWD, CPR>, grid, dim3(256), a, name, bytes, 1);
}

// normalise / input gradient from per-channel coefficients: the column-resident kernel where the chunk columns
// split into groups of 8, 16 or 32 (TCH_BN_APPLY_COLS=0: always the flat kernel)
template <typename T, int BWD>
int launch_apply_t(Context* ctx, ApplyArgs& a, const char* name, double bytes) {
  static const bool cols = [] {
    const char* e = getenv("TCH_BN_APPLY_COLS");
    return !(e && atoi(e) == 0);
  }();
  const int64_t cc = a.div_cc.d;
  a.rows = a.chunks / cc;
  if (cols && cc % 8 == 0 && a.rows >= 1024) {
    if (cc % 32 == 0) return launch_apply_cols<T, BWD, 32>(ctx, a, name, bytes);
    if (cc % 16 == 0) return launch_apply_cols<T, BWD, 16>(ctx, a, name, bytes);
    return launch_apply_cols<T, BWD, 8>(ctx, a, name, bytes);
  }
  return launch(ctx, bn_apply_kernel<T, BWD>, dim3(apply_blocks(a.chunks)), dim3(256), a, name, bytes, 1);
}

int launch_apply(Context* ctx, int dtype, bool bwd, ApplyArgs& a, double bytes) {
  if (dtype == kBF16)
    return bwd ? launch_apply_t<bf16, 1>(ctx, a, "bn_apply_kernel<bf16,bwd>", bytes)
               : launch_apply_t<bf16, 0>(ctx, a, "bn_apply_kernel<bf16,fwd>", bytes);
  return bwd ? launch_apply_t<float, 1>(ctx, a, "bn_apply_kernel<f32,bwd>", bytes)
             : launch_apply_t<float, 0>(ctx, a, "bn_apply_kernel<f32,fwd>", bytes);
}

// Inference-mode BatchNorm as one scale and one shift per channel, from the running statistics:
// y = (x - running_mean) / sqrt(running_var + eps) * gamma + beta = x * scale + shift.
struct EvalCoefArgs {
  const float* gamma;
  const float* beta;
  const float* mean;
  const float* var;
  float* coef;   // scale[C], then shift[C]
  int C;
  float eps;
};

__global__ void bn_eval_coef_kernel(EvalCoefArgs a) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.C) return;
  const float scale = a.gamma[c] / sqrtf(a.var[c] + a.eps);
  a.coef[c] = scale;
  a.coef[a.C + c] = a.beta[c] - a.mean[c] * scale;
}

int check_common(int64_t rows, int C, int dtype) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "bn: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(rows > 0 && C > 0 && C % E == 0, "bn: C must be a positive multiple of a 16-byte chunk");
  return 0;
}

}  // namespace

int bn_partial_rows(int64_t rows, int C, int dtype) { return geometry(rows, C, dtype).row_blocks; }

int64_t bn_workspace_bytes(int64_t rows, int C, int dtype) {
  Geometry g = geometry(rows, C, dtype);
  return (static_cast<int64_t>(g.row_blocks) * C * 2 + 3ll * C) * 4;
}

int bn_fwd_train(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows, int C,
                 const float* gamma, const float* beta, float* running_mean, float* running_var, float* save_mean,
                 float* save_invstd, float momentum, float eps, float* workspace) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(x && y && gamma && beta && save_mean && save_invstd && workspace, "bn_fwd_train: null tensor");
  TCH_CHECK_ARG((running_mean == nullptr) == (running_var == nullptr), "bn_fwd_train: running stats come in pairs");
  Geometry g = geometry(rows, C, dtype);
  float* partial = workspace;
  float* scale = workspace + static_cast<int64_t>(g.row_blocks) * C * 2;
  float* shift = scale + C;
  ColReduceArgs r{x, nullptr, nullptr, nullptr, nullptr, partial, rows, C, g.cc, g.ccb, g.rowlanes, g.rows_per_block};
  dim3 grid(g.col_blocks, g.row_blocks);
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double tensor_bytes = static_cast<double>(rows) * C * eb;
  int rc = dtype == kBF16 ? launch(ctx, col_reduce_kernel<bf16, 0>, grid, dim3(256), r, "bn_stats_kernel<bf16>", tensor_bytes, 1)
                          : launch(ctx, col_reduce_kernel<float, 0>, grid, dim3(256), r, "bn_stats_kernel<f32>", tensor_bytes, 1);
  if (rc) return rc;
  FwdFinalizeArgs f{partial, g.row_blocks, C, rows, gamma, beta, running_mean, running_var, save_mean, save_invstd,
                    scale,   shift,        momentum, eps};
  rc = launch(ctx, bn_fwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_fwd_finalize_kernel",
              8.0 * g.row_blocks * C, 1);
  if (rc) return rc;
  ApplyArgs a{x, residual, nullptr, y, scale, shift, nullptr, rows * g.cc, FastDiv(g.cc), relu};
  const double apply_bytes = tensor_bytes * (residual ? 3.0 : 2.0);
  return launch_apply(ctx, dtype, false, a, apply_bytes);
}

int bn_fwd_finalize(Context* ctx, const float* partial, int row_blocks, int C, int64_t rows, const float* gamma,
                    const float* beta, float* running_mean, float* running_var, float* save_mean, float* save_invstd,
                    float* coef, float momentum, float eps) {
  TCH_CHECK_ARG(partial && gamma && beta && save_mean && save_invstd && coef && row_blocks >= 1 && C > 0 && rows > 0,
                "bn_fwd_finalize: bad arguments");
  TCH_CHECK_ARG((running_mean == nullptr) == (running_var == nullptr), "bn_fwd_finalize: running stats come in pairs");
  FwdFinalizeArgs f{partial, row_blocks, C, rows, gamma, beta, running_mean, running_var, save_mean, save_invstd,
                    coef,    coef + C,   momentum, eps};
  return launch(ctx, bn_fwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_fwd_finalize_kernel",
                8.0 * row_blocks * C, 1);
}

int bn_bwd_finalize(Context* ctx, const float* partial, int row_blocks, int C, int64_t rows, const float* gamma,
                    const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta, float* coef,
                    int accumulate) {
  TCH_CHECK_ARG(partial && gamma && save_mean && save_invstd && dgamma && dbeta && coef && row_blocks >= 1 && C > 0 &&
                    rows > 0,
                "bn_bwd_finalize: bad arguments");
  BwdFinalizeArgs f{partial, row_blocks, C, rows, gamma, save_mean, save_invstd, dgamma, dbeta, coef, accumulate};
  return launch(ctx, bn_bwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_bwd_finalize_kernel",
                8.0 * row_blocks * C, 1);
}

int bn_apply_fwd(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows, int C,
                 const float* coef) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(x && y && coef, "bn_apply_fwd: null tensor");
  Geometry g = geometry(rows, C, dtype);
  const double tensor_bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 2.0 : 4.0);
  ApplyArgs a{x, residual, nullptr, y, coef, coef + C, nullptr, rows * g.cc, FastDiv(g.cc), relu};
  const double apply_bytes = tensor_bytes * (residual ? 3.0 : 2.0);
  return launch_apply(ctx, dtype, false, a, apply_bytes);
}

int bn_eval_coef(Context* ctx, const float* gamma, const float* beta, const float* running_mean,
                 const float* running_var, float* coef, int C, float eps) {
  TCH_CHECK_ARG(gamma && beta && running_mean && running_var && coef && C > 0, "bn_eval_coef: null tensor or no channels");
  EvalCoefArgs a{gamma, beta, running_mean, running_var, coef, C, eps};
  return launch(ctx, bn_eval_coef_kernel, dim3((C + 255) / 256), dim3(256), a, "bn_eval_coef_kernel", 24.0 * C, 1);
}

int bn_apply_bwd(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                 const float* coef) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(g && x && dx && coef, "bn_apply_bwd: null tensor");
  Geometry geo = geometry(rows, C, dtype);
  const double tensor_bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 2.0 : 4.0);
  ApplyArgs a{g, nullptr, x, dx, coef, coef + C, coef + 2 * C, rows * geo.cc, FastDiv(geo.cc), 0};
  return launch_apply(ctx, dtype, true, a, tensor_bytes * 3.0);
}

int bn_fwd_train_partials(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                          int64_t rows, int C, const float* gamma, const float* beta, float* running_mean,
                          float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                          const float* partial, int row_blocks, float* scratch) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(x && y && gamma && beta && save_mean && save_invstd && partial && scratch,
                "bn_fwd_train_partials: null tensor");
  TCH_CHECK_ARG(row_blocks >= 1, "bn_fwd_train_partials: no partial statistics");
  TCH_CHECK_ARG((running_mean == nullptr) == (running_var == nullptr), "bn_fwd_train: running stats come in pairs");
  const double eb0 = dtype == kBF16 ? 2.0 : 4.0;
  if (use_fused_finalize() && row_blocks <= kFusedMaxRowBlocks && C % kFusedCols == 0) {
    FinApplyArgs a{partial, row_blocks, C,        rows,    gamma,   beta, running_mean, running_var,
                   save_mean, save_invstd, nullptr, nullptr, momentum, eps,  0,            x,
                   residual, y,           relu,    fused_rows_per_slab(rows, C)};
    const dim3 grid(C / kFusedCols, static_cast<unsigned>((rows + a.rows_per_slab - 1) / a.rows_per_slab));
    const double bytes = static_cast<double>(rows) * C * eb0 * (residual ? 3.0 : 2.0);
    return dtype == kBF16 ? launch(ctx, bn_fin_apply_kernel<bf16, 0>, grid, dim3(256), a, "bn_fin_apply_kernel<bf16,fwd>", bytes, 1)
                          : launch(ctx, bn_fin_apply_kernel<float, 0>, grid, dim3(256), a, "bn_fin_apply_kernel<f32,fwd>", bytes, 1);
  }
  Geometry g = geometry(rows, C, dtype);
  float* scale = scratch;
  float* shift = scratch + C;
  FwdFinalizeArgs f{partial, row_blocks, C, rows, gamma, beta, running_mean, running_var, save_mean, save_invstd,
                    scale,   shift,      momentum, eps};
  int rc = launch(ctx, bn_fwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_fwd_finalize_kernel",
                  8.0 * row_blocks * C, 1);
  if (rc) return rc;
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double tensor_bytes = static_cast<double>(rows) * C * eb;
  ApplyArgs a{x, residual, nullptr, y, scale, shift, nullptr, rows * g.cc, FastDiv(g.cc), relu};
  const double apply_bytes = tensor_bytes * (residual ? 3.0 : 2.0);
  return launch_apply(ctx, dtype, false, a, apply_bytes);
}

int bn_bwd(Context* ctx, int dtype, const void* dy, const void* relu_mask, const void* x, void* dx, int64_t rows,
           int C, const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
           int accumulate, float* workspace) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(dy && x && dx && gamma && save_mean && save_invstd && dgamma && dbeta && workspace,
                "bn_bwd: null tensor");
  Geometry g = geometry(rows, C, dtype);
  float* partial = workspace;
  float* coef = workspace + static_cast<int64_t>(g.row_blocks) * C * 2;
  ColReduceArgs r{dy, relu_mask, x, save_mean, save_invstd, partial, rows, C, g.cc, g.ccb, g.rowlanes, g.rows_per_block};
  dim3 grid(g.col_blocks, g.row_blocks);
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double tensor_bytes = static_cast<double>(rows) * C * eb;
  const double in_tensors = relu_mask ? 3.0 : 2.0;
  int rc = dtype == kBF16 ? launch(ctx, col_reduce_kernel<bf16, 1>, grid, dim3(256), r, "bn_bwd_reduce_kernel<bf16>",
                                   tensor_bytes * in_tensors, 1)
                          : launch(ctx, col_reduce_kernel<float, 1>, grid, dim3(256), r, "bn_bwd_reduce_kernel<f32>",
                                   tensor_bytes * in_tensors, 1);
  if (rc) return rc;
  BwdFinalizeArgs f{partial, g.row_blocks, C, rows, gamma, save_mean, save_invstd, dgamma, dbeta, coef, accumulate};
  rc = launch(ctx, bn_bwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_bwd_finalize_kernel",
              8.0 * g.row_blocks * C, 1);
  if (rc) return rc;
  ApplyArgs a{dy, relu_mask, x, dx, coef, coef + C, coef + 2 * C, rows * g.cc, FastDiv(g.cc), 0};
  return launch_apply(ctx, dtype, true, a, tensor_bytes * (in_tensors + 1.0));
}

int bn_bwd_partials(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                    const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma,
                    float* dbeta, int accumulate, const float* partial, int row_blocks, float* scratch) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(g && x && dx && gamma && save_mean && save_invstd && dgamma && dbeta && partial && scratch,
                "bn_bwd_partials: null tensor");
  TCH_CHECK_ARG(row_blocks >= 1, "bn_bwd_partials: no partial sums");
  if (use_fused_finalize() && row_blocks <= kFusedMaxRowBlocks && C % kFusedCols == 0) {
    FinApplyArgs a{partial, row_blocks, C, rows, gamma, nullptr, nullptr, nullptr, const_cast<float*>(save_mean),
                   const_cast<float*>(save_invstd), dgamma, dbeta, 0.f, 0.f, accumulate, g, x, dx, 0,
                   fused_rows_per_slab(rows, C)};
    const dim3 grid(C / kFusedCols, static_cast<unsigned>((rows + a.rows_per_slab - 1) / a.rows_per_slab));
    const double bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 2.0 : 4.0) * 3.0;
    return dtype == kBF16 ? launch(ctx, bn_fin_apply_kernel<bf16, 1>, grid, dim3(256), a, "bn_fin_apply_kernel<bf16,bwd>", bytes, 1)
                          : launch(ctx, bn_fin_apply_kernel<float, 1>, grid, dim3(256), a, "bn_fin_apply_kernel<f32,bwd>", bytes, 1);
  }
  Geometry geo = geometry(rows, C, dtype);
  float* coef = scratch;
  BwdFinalizeArgs f{partial, row_blocks, C, rows, gamma, save_mean, save_invstd, dgamma, dbeta, coef, accumulate};
  int rc = launch(ctx, bn_bwd_finalize_kernel, dim3((C + 7) / 8), dim3(kFinalizeThreads), f, "bn_bwd_finalize_kernel",
                  8.0 * row_blocks * C, 1);
  if (rc) return rc;
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double tensor_bytes = static_cast<double>(rows) * C * eb;
  ApplyArgs a{g, nullptr, x, dx, coef, coef + C, coef + 2 * C, rows * geo.cc, FastDiv(geo.cc), 0};
  return launch_apply(ctx, dtype, true, a, tensor_bytes * 3.0);
}

int bn_fwd_train_acc(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows,
                     int C, const float* gamma, const float* beta, float* running_mean, float* running_var,
                     float* save_mean, float* save_invstd, float momentum, float eps, const long long* acc,
                     int acc_copies) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(x && y && gamma && beta && save_mean && save_invstd && acc, "bn_fwd_train_acc: null tensor");
  TCH_CHECK_ARG((running_mean == nullptr) == (running_var == nullptr), "bn_fwd_train_acc: running stats come in pairs");
  TCH_CHECK_ARG(C % (dtype == kBF16 ? 64 : 32) == 0, "bn_fwd_train_acc: channels must come in groups of eight 16-byte chunks");
  TCH_CHECK_ARG(acc_copies >= 1 && (acc_copies & (acc_copies - 1)) == 0, "bn_fwd_train_acc: copies must be a power of two");
  AccApplyArgs a{acc, acc_copies, C, rows, gamma, beta, running_mean, running_var, save_mean, save_invstd, nullptr, nullptr,
                 momentum, eps, 0, x, residual, y, relu, 0, 0};
  const double bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 2.0 : 4.0) * (residual ? 3.0 : 2.0);
  return dtype == kBF16 ? launch_acc_apply_t<bf16, 0>(ctx, a, "bn_acc_apply_kernel<bf16,fwd>", bytes)
                        : launch_acc_apply_t<float, 0>(ctx, a, "bn_acc_apply_kernel<f32,fwd>", bytes);
}

int bn_bwd_acc(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
               const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
               int accumulate, const long long* acc, int acc_copies) {
  if (int rc = check_common(rows, C, dtype)) return rc;
  TCH_CHECK_ARG(g && x && dx && gamma && save_mean && save_invstd && dgamma && dbeta && acc, "bn_bwd_acc: null tensor");
  TCH_CHECK_ARG(C % (dtype == kBF16 ? 64 : 32) == 0, "bn_bwd_acc: channels must come in groups of eight 16-byte chunks");
  TCH_CHECK_ARG(acc_copies >= 1 && (acc_copies & (acc_copies - 1)) == 0, "bn_bwd_acc: copies must be a power of two");
  AccApplyArgs a{acc, acc_copies, C, rows, gamma, nullptr, nullptr, nullptr, const_cast<float*>(save_mean),
                 const_cast<float*>(save_invstd), dgamma, dbeta, 0.f, 0.f, accumulate, g, x, dx, 0, 0, 0};
  const double bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 2.0 : 4.0) * 3.0;
  return dtype == kBF16 ? launch_acc_apply_t<bf16, 1>(ctx, a, "bn_acc_apply_kernel<bf16,bwd>", bytes)
                        : launch_acc_apply_t<float, 1>(ctx, a, "bn_acc_apply_kernel<f32,bwd>", bytes);
}

}  // namespace tch
