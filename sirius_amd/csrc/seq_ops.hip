// Row-wise and elementwise operators of the transformer training steps (Swin-B, GPT-2):
// LayerNorm, GELU (exact erf and the tanh form), attention softmax (scale, additive bias,
// window mask, causal), AdamW with a bf16 shadow copy, token + position embedding.
// All HBM-bound: 16-byte chunks per lane, one wavefront per row for the row-wise ones.
//
// Restated arithmetic and its reference call sites (the arithmetic itself lives in PyTorch /
// torchvision / transformers, which the reference calls):
//   nn.LayerNorm(eps 1e-5), nn.GELU, window attention softmax with relative position bias
//   and the shift mask                        train/swin_b_tiny.py:8-172, train/swin_b.py:38
//   GPT-2 gelu_new, causal attention, wte + wpe   train/gpt2.py:26
//   torch.optim.AdamW                         train/gpt2.py:31, train/swin_b.py:43 (variants)
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

unsigned flat_blocks(int64_t items, int64_t cap = 1 << 20) {
  int64_t b = (items + 255) / 256;
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return static_cast<unsigned>(b);
}

// ---------------------------------------------------------------------------
// LayerNorm over the last dimension of [rows, C]
// ---------------------------------------------------------------------------
constexpr int kLnMaxC = 2048;  // longest row: a lane holds 32 elements of it

struct LnArgs {
  const void* x;
  const void* dy;  // backward
  const void* add; // backward, optional: added to dx (the residual branch's gradient)
                   // forward, optional: added to x before anything else; the sum, rounded to T, goes to sum_out
  void* sum_out;   // forward with add: x + add in row order
  void* out;       // forward: y   backward: dx
  const float* gamma;
  const float* beta;
  float* mean;   // [rows]  forward: written   backward: read
  float* rstd;   // [rows]
  float* partial;  // backward: [gridDim.x][C][2] = per-workgroup (sum dy*xhat, sum dy)
  int64_t rows;
  int C, cc;
  int rows_per_wg;
  float eps;
  // Optional window order (Swin): rows are the pixels of [B, win_h, win_w] images; a tensor flagged below is laid
  // out as window tokens instead (cyclic shift by -win_shift, then win_ws x win_ws windows) and is reached through
  // window_row().  win_ws == 0: every tensor is in row order.  Where the window does not tile the image the window
  // tokens live in the frame padded at the bottom and the right to win_hp x win_wp (whole windows): a window-ordered
  // tensor then has B * win_hp * win_wp rows, of which these kernels touch the ones that belong to pixels.
  int win_h, win_w, win_ws, win_shift;
  int win_hp, win_wp;
  int win_out;   // forward: y   backward: dx
  int win_dy;    // backward: dy
  int win_add;   // backward: the addend
};

// pixel row (b, h, w) -> its window token (b, wh, ww, i, j): h - shift = wh * ws + i, w - shift = ww * ws + j, modulo
// the (padded) frame
__device__ inline int64_t window_row(const LnArgs& p, int64_t row) {
  const int w = static_cast<int>(row % p.win_w);
  int64_t t = row / p.win_w;
  const int h = static_cast<int>(t % p.win_h);
  t /= p.win_h;
  int hs = h - p.win_shift, wsft = w - p.win_shift;
  if (hs < 0) hs += p.win_hp;
  if (wsft < 0) wsft += p.win_wp;
  const int wh = hs / p.win_ws, i = hs - wh * p.win_ws, ww = wsft / p.win_ws, j = wsft - ww * p.win_ws;
  return (((t * (p.win_hp / p.win_ws) + wh) * (p.win_wp / p.win_ws) + ww) * p.win_ws + i) * p.win_ws + j;
}

// L lanes per row (L = 64: one wavefront per row, NCH 16-byte chunks per lane; L = 16 or 32: short rows, 64 / L
// rows per wavefront, one chunk per lane); the row stays in registers between the passes
template <int L>
__device__ inline float row_sum(float v) {
#pragma unroll
  for (int off = L / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <typename T>
__device__ inline void load_params(const float* src, int c, float* out) {
  constexpr int E = Elem<T>::kPerChunk;
#pragma unroll
  for (int e = 0; e < E; e += 4) {
    const float4 t = *reinterpret_cast<const float4*>(src + c * E + e);
    out[e] = t.x;
    out[e + 1] = t.y;
    out[e + 2] = t.z;
    out[e + 3] = t.w;
  }
}

template <typename T, int NCH, int L>
__global__ __launch_bounds__(256) void ln_fwd_kernel(LnArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int RPW = 64 / L;   // rows per wavefront
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % L;
  const int64_t row = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * RPW + lane / L;
  const bool live = row < p.rows;
  const uint4* src = static_cast<const uint4*>(p.x) + row * p.cc;
  const int64_t wrow = (live && p.win_ws) ? window_row(p, row) : row;
  float v[NCH][E];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = sub + j * L;
    if (live && c < p.cc) {
      Chunk ch;
      ch.u = src[c];
      chunk_to_float<T>(ch, v[j]);
      if (p.add) {
        // the residual sum of a block: rounded to T as the separate addition would leave it, kept for later
        Chunk ca;
        ca.u = (static_cast<const uint4*>(p.add) + (p.win_add ? wrow : row) * p.cc)[c];
        float a[E];
        chunk_to_float<T>(ca, a);
#pragma unroll
        for (int e = 0; e < E; ++e) v[j][e] += a[e];
        ch = float_to_chunk<T>(v[j]);
        chunk_to_float<T>(ch, v[j]);
        (static_cast<uint4*>(p.sum_out) + row * p.cc)[c] = ch.u;
      }
#pragma unroll
      for (int e = 0; e < E; ++e) s += v[j][e];
    }
  }
  const float mean = row_sum<L>(s) / static_cast<float>(p.C);
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    if (live && sub + j * L < p.cc) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const float d = v[j][e] - mean;
        q += d * d;
      }
    }
  }
  const float rstd = 1.0f / sqrtf(row_sum<L>(q) / static_cast<float>(p.C) + p.eps);
  if (!live) return;
  if (sub == 0) {
    p.mean[row] = mean;
    p.rstd[row] = rstd;
  }
  uint4* dst = static_cast<uint4*>(p.out) + (p.win_out ? wrow : row) * p.cc;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = sub + j * L;
    if (c < p.cc) {
      float o[E], ga[E], be[E];
      load_params<T>(p.gamma, c, ga);
      load_params<T>(p.beta, c, be);
#pragma unroll
      for (int e = 0; e < E; ++e) o[e] = (v[j][e] - mean) * rstd * ga[e] + be[e];
      dst[c] = float_to_chunk<T>(o).u;
    }
  }
}

// dx per row; the column sums for dgamma / dbeta are kept per lane over the rows its row group walks, then
// summed over the 4 * 64 / L row groups of the workgroup through LDS: one partial row per workgroup
template <typename T, int NCH, int L>
__global__ __launch_bounds__(256) void ln_bwd_kernel(LnArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int RPW = 64 / L;
  constexpr int GROUPS = 4 * RPW;
  constexpr int COLS = NCH * L * E;      // columns a row group covers
  __shared__ float red[GROUPS][COLS * 2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % L, group = wave * RPW + lane / L;
  float dg[NCH][E], db[NCH][E], gam[NCH][E];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = sub + j * L;
#pragma unroll
    for (int e = 0; e < E; ++e) dg[j][e] = db[j][e] = gam[j][e] = 0.f;
    if (c < p.cc) load_params<T>(p.gamma, c, gam[j]);
  }
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * p.rows_per_wg;
  int64_t r1 = r0 + p.rows_per_wg;
  if (r1 > p.rows) r1 = p.rows;
  const float inv_c = 1.0f / static_cast<float>(p.C);
  // rows_per_wg is a multiple of GROUPS, so the groups of a wavefront stay in step (the row sums below are
  // taken by all lanes); a group beyond the last row works on nothing.  A group takes R rows per trip and
  // requests the chunks of all of them before it uses any.  R = 1: two rows per trip cost 36 registers more
  // (161 against 125 for rows of 768), and beside the weight gradients of the second lane, which leave room for
  // one such wave per SIMD, the kernel was slower for it (GPT-2: 40.7 against 36.5 us per launch in the step).
  constexpr int R = 1;
  for (int64_t base = r0; base < r1; base += R * GROUPS) {
    bool live[R];
    int64_t wrows[R];
    float mean[R], rstd[R];
    Chunk cx[R][NCH], cg[R][NCH], cr[R][NCH];
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const int64_t row = base + q * GROUPS + group;
      live[q] = row < r1;
      mean[q] = rstd[q] = 0.f;
      int64_t wrow = row;
      if (live[q]) {
        mean[q] = p.mean[row];
        rstd[q] = p.rstd[row];
        if (p.win_ws) wrow = window_row(p, row);
      }
      wrows[q] = wrow;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const int c = sub + j * L;
        cx[q][j] = cg[q][j] = cr[q][j] = zero_chunk();
        if (live[q] && c < p.cc) {
          cx[q][j].u = (static_cast<const uint4*>(p.x) + row * p.cc)[c];
          cg[q][j].u = (static_cast<const uint4*>(p.dy) + (p.win_dy ? wrow : row) * p.cc)[c];
          if (p.add) cr[q][j].u = (static_cast<const uint4*>(p.add) + (p.win_add ? wrow : row) * p.cc)[c];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const int64_t row = base + q * GROUPS + group;
      float xh[NCH][E], g[NCH][E];
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const int c = sub + j * L;
        chunk_to_float<T>(cx[q][j], xh[j]);
        chunk_to_float<T>(cg[q][j], g[j]);
        if (live[q] && c < p.cc) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            xh[j][e] = (xh[j][e] - mean[q]) * rstd[q];
            dg[j][e] += g[j][e] * xh[j][e];
            db[j][e] += g[j][e];
            g[j][e] *= gam[j][e];
            a += g[j][e];
            b += g[j][e] * xh[j][e];
          }
        }
      }
      a = row_sum<L>(a) * inv_c;
      b = row_sum<L>(b) * inv_c;
      if (!live[q]) continue;
      uint4* dst = static_cast<uint4*>(p.out) + (p.win_out ? wrows[q] : row) * p.cc;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const int c = sub + j * L;
        if (c < p.cc) {
          float o[E];
#pragma unroll
          for (int e = 0; e < E; ++e) o[e] = rstd[q] * (g[j][e] - a - xh[j][e] * b);
          if (p.add) {
            float r[E];
            chunk_to_float<T>(cr[q][j], r);
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += r[e];
          }
          dst[c] = float_to_chunk<T>(o).u;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NCH; ++j)
#pragma unroll
    for (int e = 0; e < E; ++e) {
      red[group][((j * L + sub) * E + e) * 2] = dg[j][e];
      red[group][((j * L + sub) * E + e) * 2 + 1] = db[j][e];
    }
  __syncthreads();
  // column col lives at chunk c = col / E = j * L + sub, element col % E: position col of a group's row
  for (int col = threadIdx.x; col < p.C; col += 256) {
    float sg = 0.f, sb = 0.f;
#pragma unroll
    for (int gidx = 0; gidx < GROUPS; ++gidx) {
      sg += red[gidx][col * 2];
      sb += red[gidx][col * 2 + 1];
    }
    float2* dst = reinterpret_cast<float2*>(p.partial + (static_cast<int64_t>(blockIdx.x) * p.C + col) * 2);
    *dst = make_float2(sg, sb);
  }
}

struct ColSumArgs {
  const float* partial;  // [blocks][C][2]
  float* out0;           // (+)= sum_b partial[b][c][0]
  float* out1;           // (+)= sum_b partial[b][c][1]
  int blocks, C, accumulate;
};

// 8 columns x 32 lanes per workgroup, fp64 sums in a fixed order
__global__ __launch_bounds__(256) void col_sum_kernel(ColSumArgs p) {
  __shared__ double red[32][8][2];
  const int cl = threadIdx.x & 7, lane = threadIdx.x >> 3;
  const int c = blockIdx.x * 8 + cl;
  double s = 0.0, q = 0.0;
  if (c < p.C) {
    constexpr int U = 8;
    for (int b = lane; b < p.blocks; b += U * 32) {
      float2 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int bb = b + u * 32;
        v[u] = bb < p.blocks ? *reinterpret_cast<const float2*>(p.partial + (static_cast<int64_t>(bb) * p.C + c) * 2)
                             : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        s += v[u].x;
        q += v[u].y;
      }
    }
  }
  red[lane][cl][0] = s;
  red[lane][cl][1] = q;
  __syncthreads();
  for (int off = 16; off > 0; off >>= 1) {
    if (lane < off) {
      red[lane][cl][0] += red[lane + off][cl][0];
      red[lane][cl][1] += red[lane + off][cl][1];
    }
    __syncthreads();
  }
  if (lane == 0 && c < p.C) {
    const float a = static_cast<float>(red[0][cl][0]), b = static_cast<float>(red[0][cl][1]);
    p.out0[c] = p.accumulate ? p.out0[c] + a : a;
    p.out1[c] = p.accumulate ? p.out1[c] + b : b;
  }
}

// ---------------------------------------------------------------------------
// GELU
// ---------------------------------------------------------------------------
struct GeluArgs {
  const void* x;
  const void* dy;  // backward
  void* out;
  int64_t chunks;
  int tanh_form;
};

__device__ inline float gelu_value(float x, int tanh_form) {
  if (tanh_form) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + tanhf(u));
  }
  return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
}

__device__ inline float gelu_slope(float x, int tanh_form) {
  if (tanh_form) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float t = tanhf(u);
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * 0.7978845608028654f * (1.0f + 3.0f * 0.044715f * x * x);
  }
  return 0.5f * (1.0f + erff(x * 0.7071067811865476f)) + x * 0.3989422804014327f * expf(-0.5f * x * x);
}

template <typename T, int BWD>
__global__ __launch_bounds__(256) void gelu_kernel(GeluArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < p.chunks; i += stride) {
    Chunk cx;
    cx.u = load_streaming_u4(p.x, i);
    float x[E], o[E];
    chunk_to_float<T>(cx, x);
    if (BWD) {
      Chunk cg;
      cg.u = load_streaming_u4(p.dy, i);
      float g[E];
      chunk_to_float<T>(cg, g);
#pragma unroll
      for (int e = 0; e < E; ++e) o[e] = g[e] * gelu_slope(x[e], p.tanh_form);
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e) o[e] = gelu_value(x[e], p.tanh_form);
    }
    static_cast<uint4*>(p.out)[i] = float_to_chunk<T>(o).u;
  }
}

// ---------------------------------------------------------------------------
// attention softmax over rows of [batch, heads, Lq, Lk]
// ---------------------------------------------------------------------------
struct SoftmaxArgs {
  const void* s;      // forward: scores        backward: probabilities
  const void* dp;     // backward: gradient of the probabilities
  void* out;          // forward: probabilities backward: gradient of the scores
  const float* bias;  // optional [heads][Lq][Lk], added after scaling
  const float* mask;  // optional [windows][Lq][Lk], added after scaling; window = batch % windows
  int64_t rows;       // batch * heads * Lq
  int heads, Lq, Lk, windows, causal;
  float scale;
};

// one wavefront per row, four rows per workgroup
template <typename T, int BWD>
__global__ __launch_bounds__(256) void attn_softmax_kernel(SoftmaxArgs p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  if (row >= p.rows) return;
  const T* src = static_cast<const T*>(p.s) + row * p.Lk;
  T* dst = static_cast<T*>(p.out) + row * p.Lk;
  if (BWD) {
    // causal: probabilities beyond the query's own position are zero and dp there is never read (it
    // may be unwritten memory)
    const int i = static_cast<int>(row % p.Lq);
    const int limit = p.causal ? (i + 1 < p.Lk ? i + 1 : p.Lk) : p.Lk;
    const T* dp = static_cast<const T*>(p.dp) + row * p.Lk;
    float dot = 0.f;
    for (int j = lane; j < limit; j += 64) dot += Elem<T>::load(src + j) * Elem<T>::load(dp + j);
    dot = wave_sum(dot);
    for (int j = lane; j < p.Lk; j += 64)
      Elem<T>::store(dst + j, j < limit ? p.scale * Elem<T>::load(src + j) * (Elem<T>::load(dp + j) - dot) : 0.f);
    return;
  }
  const int i = static_cast<int>(row % p.Lq);
  const int64_t bh = row / p.Lq;
  const int h = static_cast<int>(bh % p.heads);
  const int64_t b = bh / p.heads;
  const float* bias = p.bias ? p.bias + (static_cast<int64_t>(h) * p.Lq + i) * p.Lk : nullptr;
  const float* mask = p.mask ? p.mask + (static_cast<int64_t>(b % p.windows) * p.Lq + i) * p.Lk : nullptr;
  const int limit = p.causal ? (i + 1 < p.Lk ? i + 1 : p.Lk) : p.Lk;  // keys [0, limit) take part
  auto logit = [&](int j) {
    float v = Elem<T>::load(src + j) * p.scale;
    if (bias) v += bias[j];
    if (mask) v += mask[j];
    return v;
  };
  float mx = -INFINITY;
  for (int j = lane; j < limit; j += 64) mx = fmaxf(mx, logit(j));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < limit; j += 64) sum += expf(logit(j) - mx);
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (int j = lane; j < p.Lk; j += 64) Elem<T>::store(dst + j, j < limit ? expf(logit(j) - mx) * inv : 0.f);
}

// ---------------------------------------------------------------------------
// AdamW over a flat fp32 parameter buffer with a bf16 shadow
// ---------------------------------------------------------------------------
struct AdamTickArgs {
  int* step;       // device step counter, incremented here
  float* scalars;  // [0] = 1 - beta1^t, [1] = sqrt(1 - beta2^t)
  double beta1, beta2;
};

__global__ void adamw_tick_kernel(AdamTickArgs p) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const int t = *p.step + 1;
  *p.step = t;
  p.scalars[0] = static_cast<float>(1.0 - pow(p.beta1, static_cast<double>(t)));
  p.scalars[1] = static_cast<float>(sqrt(1.0 - pow(p.beta2, static_cast<double>(t))));
}

struct AdamArgs {
  float* param;
  const float* grad;
  float* m;
  float* v;
  uint16_t* shadow;
  const float* scalars;
  int64_t n;
  // every constant is rounded to fp32 once, from the double the caller gave (1 - beta as well:
  // 1 - 0.999f is off by 1e-5 relative)
  float lr, beta2, one_minus_beta1, one_minus_beta2, eps, decay;
  int aligned;   // every buffer starts on a 16-byte boundary (the shadow on 8): 16-byte accesses are in order
};

__device__ inline void adamw_element(const AdamArgs& p, float step_size, float bc2_sqrt, float g, float& w, float& m,
                                     float& v) {
  w *= p.decay;
  m = m + (g - m) * p.one_minus_beta1;
  v = v * p.beta2 + p.one_minus_beta2 * g * g;
  const float denom = sqrtf(v) / bc2_sqrt + p.eps;
  w -= step_size * (m / denom);
}

// four elements per thread and trip, 16-byte streaming accesses; the last n % 4 elements one by one
__global__ __launch_bounds__(256) void adamw_kernel(AdamArgs p) {
  const float bc1 = p.scalars[0], bc2_sqrt = p.scalars[1];
  const float step_size = p.lr / bc1;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; i < p.n; i += stride) {
    if (p.aligned && i + 4 <= p.n) {
      const float4 g = load_streaming_f4(p.grad + i);
      float4 w = load_streaming_f4(p.param + i);
      float4 m = load_streaming_f4(p.m + i);
      float4 v = load_streaming_f4(p.v + i);
      adamw_element(p, step_size, bc2_sqrt, g.x, w.x, m.x, v.x);
      adamw_element(p, step_size, bc2_sqrt, g.y, w.y, m.y, v.y);
      adamw_element(p, step_size, bc2_sqrt, g.z, w.z, m.z, v.z);
      adamw_element(p, step_size, bc2_sqrt, g.w, w.w, m.w, v.w);
      store_streaming_f4(p.param + i, w);
      store_streaming_f4(p.m + i, m);
      store_streaming_f4(p.v + i, v);
      if (p.shadow) {
        uint2 sh;
        sh.x = float_to_bf16_bits(w.x) | (static_cast<uint32_t>(float_to_bf16_bits(w.y)) << 16);
        sh.y = float_to_bf16_bits(w.z) | (static_cast<uint32_t>(float_to_bf16_bits(w.w)) << 16);
        *reinterpret_cast<uint2*>(p.shadow + i) = sh;
      }
    } else {
      for (int64_t j = i; j < p.n && j < i + 4; ++j) {
        float w = p.param[j], m = p.m[j], v = p.v[j];
        adamw_element(p, step_size, bc2_sqrt, p.grad[j], w, m, v);
        p.param[j] = w;
        p.m[j] = m;
        p.v[j] = v;
        if (p.shadow) p.shadow[j] = float_to_bf16_bits(w);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// token + position embedding
// ---------------------------------------------------------------------------
struct EmbedArgs {
  const int64_t* ids;  // [B*T]
  const void* wte;     // [vocab][C]   (forward, T)
  const void* wpe;     // [>=T][C]
  void* out;           // [B*T][C]     (forward)
  const void* dy;      // [B*T][C]     (backward)
  float* dwte;         // [vocab][C] fp32, += (backward)
  float* dwpe;         // [T][C] fp32, (+)= (backward)
  int64_t tokens;
  int T, C, cc, vocab, B, accumulate;
  const int32_t* next_same;   // backward: chains of positions that hold the same token (nullptr: atomics)
  const int32_t* first;
};

template <typename T>
__global__ __launch_bounds__(256) void embed_fwd_kernel(EmbedArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t total = p.tokens * p.cc;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t tok = i / p.cc;
    const int c = static_cast<int>(i - tok * p.cc);
    const int t = static_cast<int>(tok % p.T);
    int64_t id = p.ids[tok];
    if (id < 0 || id >= p.vocab) id = 0;  // ids are validated on the host; never read outside the table
    Chunk a, b;
    a.u = static_cast<const uint4*>(p.wte)[id * p.cc + c];
    b.u = static_cast<const uint4*>(p.wpe)[static_cast<int64_t>(t) * p.cc + c];
    float va[E], vb[E];
    chunk_to_float<T>(a, va);
    chunk_to_float<T>(b, vb);
#pragma unroll
    for (int e = 0; e < E; ++e) va[e] += vb[e];
    static_cast<uint4*>(p.out)[i] = float_to_chunk<T>(va).u;
  }
}

// Which positions hold the same token: next_same[i] = the next position after i with ids[i] (or -1),
// first[i] = 1 when no earlier position holds it.  A workgroup owns 64 positions (one per lane); the ids pass
// through LDS in chunks of 4096 and each of the four wavefronts compares its quarter of a chunk against the
// lane's id (every lane of a wavefront reads the same LDS word: a broadcast), without branches; the four
// partial answers meet in LDS.  Ids outside the table count as 0, as in the kernels that use them.
struct ChainArgs {
  const int64_t* ids;
  int32_t* next_same;
  int32_t* first;
  int n, vocab;
};

__global__ __launch_bounds__(256) void embed_chain_kernel(ChainArgs p) {
  constexpr int kChunk = 4096;
  __shared__ int32_t s_ids[kChunk];
  __shared__ int32_t s_next[4][64];
  __shared__ int32_t s_prev[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;
  auto clamp_id = [&](int64_t v) { return (v < 0 || v >= p.vocab) ? 0 : static_cast<int32_t>(v); };
  const int32_t id = i < p.n ? clamp_id(p.ids[i]) : -1;
  int next = 0x7fffffff, prev = 0;
  for (int base = 0; base < p.n; base += kChunk) {
    const int len = min(kChunk, p.n - base);
    __syncthreads();
    for (int j = threadIdx.x; j < kChunk; j += 256) s_ids[j] = j < len ? clamp_id(p.ids[base + j]) : -2;
    __syncthreads();
    const int q0 = wave * (kChunk / 4);
    for (int j = q0; j < q0 + kChunk / 4; j += 4) {
      const int4 v = *reinterpret_cast<const int4*>(&s_ids[j]);
      const int g = base + j;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int32_t w = e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w;
        const bool same = w == id;
        prev |= (same && g + e < i) ? 1 : 0;
        next = (same && g + e > i) ? min(next, g + e) : next;
      }
    }
  }
  s_next[wave][lane] = next;
  s_prev[wave][lane] = prev;
  __syncthreads();
  if (wave == 0 && i < p.n) {
    const int nx = min(min(s_next[0][lane], s_next[1][lane]), min(s_next[2][lane], s_next[3][lane]));
    const int pv = s_prev[0][lane] | s_prev[1][lane] | s_prev[2][lane] | s_prev[3][lane];
    p.next_same[i] = nx == 0x7fffffff ? -1 : nx;
    p.first[i] = pv ? 0 : 1;
  }
}

// dwpe[t] = sum over the batch (fixed order).  dwte[id] += sum of the dy rows of the positions that hold id,
// added up in position order by the thread of the FIRST such position, which is the only writer of that row:
// no atomics, the same bits every run.  (chain == nullptr: fp32 atomics per position instead; rows that share
// a token then meet in an order that may differ between runs.)
template <typename T>
__global__ __launch_bounds__(256) void embed_bwd_kernel(EmbedArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int32_t* next_same = p.next_same;
  const int32_t* first = p.first;
  const int64_t per_batch = static_cast<int64_t>(p.T) * p.cc;
  const int64_t total = p.tokens * p.cc;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
    const int64_t tok = i / p.cc;
    const int c = static_cast<int>(i - tok * p.cc);
    if (i < per_batch) {   // position tok (< T) of every sequence: the position embedding's gradient
      float acc[E];
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = 0.f;
      for (int b = 0; b < p.B; ++b) {
        Chunk g;
        g.u = static_cast<const uint4*>(p.dy)[(static_cast<int64_t>(b) * p.T + tok) * p.cc + c];
        float v[E];
        chunk_to_float<T>(g, v);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] += v[e];
      }
      float* dst = p.dwpe + tok * p.C + c * E;
#pragma unroll
      for (int e = 0; e < E; ++e) dst[e] = p.accumulate ? dst[e] + acc[e] : acc[e];
    }
    int64_t id = p.ids[tok];
    if (id < 0 || id >= p.vocab) id = 0;
    float* row = p.dwte + id * p.C + c * E;
    if (next_same == nullptr) {
      Chunk g;
      g.u = static_cast<const uint4*>(p.dy)[i];
      float v[E];
      chunk_to_float<T>(g, v);
#pragma unroll
      for (int e = 0; e < E; ++e) atomicAdd(row + e, v[e]);
      continue;
    }
    if (!first[tok]) continue;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.f;
    for (int64_t j = tok; j >= 0; j = next_same[j]) {
      Chunk g;
      g.u = static_cast<const uint4*>(p.dy)[j * p.cc + c];
      float v[E];
      chunk_to_float<T>(g, v);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] += v[e];
    }
#pragma unroll
    for (int e = 0; e < E; ++e) row[e] += acc[e];
  }
}

int check_rows(const char* what, int dtype, int64_t rows, int C) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, std::string(what) + ": dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(rows > 0 && C > 0 && C % E == 0, std::string(what) + ": C must be a positive multiple of a 16-byte chunk");
  return 0;
}

// rows per workgroup of the backward: about 1024 workgroups, a multiple of 16 (the most rows a workgroup takes
// in one pass, with 16 lanes per row)
int ln_rows_per_wg(int64_t rows) {
  int64_t r = (rows + 1023) / 1024;
  r = (r + 15) / 16 * 16;
  return static_cast<int>(r);
}

// lanes per row and chunks per lane for rows of cc 16-byte chunks
struct LnShape {
  int lanes, nch;
};
LnShape ln_shape(int cc) {
  if (cc <= 16) return {16, 1};
  if (cc <= 32) return {32, 1};
  return {64, (cc + 63) / 64};
}

template <typename T, bool BWD>
void (*ln_kernel_for(LnShape sh))(LnArgs) {
  if (sh.lanes == 16) return BWD ? ln_bwd_kernel<T, 1, 16> : ln_fwd_kernel<T, 1, 16>;
  if (sh.lanes == 32) return BWD ? ln_bwd_kernel<T, 1, 32> : ln_fwd_kernel<T, 1, 32>;
  switch (sh.nch) {
    case 1:
      return BWD ? ln_bwd_kernel<T, 1, 64> : ln_fwd_kernel<T, 1, 64>;
    case 2:
      return BWD ? ln_bwd_kernel<T, 2, 64> : ln_fwd_kernel<T, 2, 64>;
    case 3:
      return BWD ? ln_bwd_kernel<T, 3, 64> : ln_fwd_kernel<T, 3, 64>;
    default:
      break;
  }
  if constexpr (sizeof(T) == 2) return BWD ? ln_bwd_kernel<T, 4, 64> : ln_fwd_kernel<T, 4, 64>;
  if (sh.nch <= 4) return BWD ? ln_bwd_kernel<T, 4, 64> : ln_fwd_kernel<T, 4, 64>;
  if (sh.nch <= 6) return BWD ? ln_bwd_kernel<T, 6, 64> : ln_fwd_kernel<T, 6, 64>;
  return BWD ? ln_bwd_kernel<T, 8, 64> : ln_fwd_kernel<T, 8, 64>;
}

}  // namespace

int layernorm_bwd_partial_rows(int64_t rows) {
  const int r = ln_rows_per_wg(rows);
  return static_cast<int>((rows + r - 1) / r);
}

int bind_window(LnArgs& a, const LnWindow* win, int64_t rows, int allowed) {
  if (!win || win->ws == 0) return 0;
  TCH_CHECK_ARG(win->H > 0 && win->W > 0 && win->ws > 0, "layernorm: window geometry must be positive");
  TCH_CHECK_ARG(win->shift >= 0 && win->shift < win->ws, "layernorm: shift must be in [0, window)");
  TCH_CHECK_ARG(rows % (static_cast<int64_t>(win->H) * win->W) == 0, "layernorm: rows must be whole images");
  TCH_CHECK_ARG((win->tensors & ~allowed) == 0, "layernorm: a tensor flagged as window-ordered does not exist in this direction");
  a.win_h = win->H;
  a.win_w = win->W;
  a.win_ws = win->ws;
  a.win_shift = win->shift;
  a.win_hp = (win->H + win->ws - 1) / win->ws * win->ws;
  a.win_wp = (win->W + win->ws - 1) / win->ws * win->ws;
  a.win_out = win->tensors & 1;
  a.win_dy = (win->tensors >> 1) & 1;
  a.win_add = (win->tensors >> 2) & 1;
  return 0;
}

int layernorm_fwd(Context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta, float* mean,
                  float* rstd, int64_t rows, int C, float eps, const LnWindow* win, const void* add, void* sum_out) {
  if (int rc = check_rows("layernorm_fwd", dtype, rows, C)) return rc;
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(C <= kLnMaxC, "layernorm: rows longer than 2048 elements are not supported");
  TCH_CHECK_ARG(x && y && gamma && beta && mean && rstd, "layernorm_fwd: null tensor");
  TCH_CHECK_ARG((add == nullptr) == (sum_out == nullptr), "layernorm_fwd: an addend goes with a place for the sum");
  LnArgs a{x, nullptr, add, sum_out, y, gamma, beta, mean, rstd, nullptr, rows, C, C / E, 0, eps};
  if (int rc = bind_window(a, win, rows, add ? 5 : 1)) return rc;
  TCH_CHECK_ARG(!(a.win_out && (x == y || sum_out == y)), "layernorm_fwd: a window-ordered output cannot overwrite a row-ordered tensor");
  TCH_CHECK_ARG(!(a.win_add && (sum_out == add || y == add)), "layernorm_fwd: a window-ordered addend cannot be overwritten in row order");
  const double bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 4.0 : 8.0) * (add ? 2.0 : 1.0);
  const LnShape sh = ln_shape(a.cc);
  const dim3 grid(static_cast<unsigned>((rows + 4 * (64 / sh.lanes) - 1) / (4 * (64 / sh.lanes))));
  return dtype == kBF16 ? launch(ctx, ln_kernel_for<bf16, false>(sh), grid, dim3(256), a, "ln_fwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, ln_kernel_for<float, false>(sh), grid, dim3(256), a, "ln_fwd_kernel<f32>", bytes, 1);
}

int layernorm_bwd(Context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual, const float* gamma,
                  const float* mean, const float* rstd, float* dgamma, float* dbeta, int accumulate, int64_t rows,
                  int C, float* partial, const LnWindow* win) {
  if (int rc = check_rows("layernorm_bwd", dtype, rows, C)) return rc;
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(C <= kLnMaxC, "layernorm: rows longer than 2048 elements are not supported");
  TCH_CHECK_ARG(dy && x && dx && gamma && mean && rstd && dgamma && dbeta && partial, "layernorm_bwd: null tensor");
  const int rpw = ln_rows_per_wg(rows);
  const int blocks = static_cast<int>((rows + rpw - 1) / rpw);
  LnArgs a{x,    dy,   residual, nullptr, dx,  gamma, nullptr, const_cast<float*>(mean), const_cast<float*>(rstd),
           partial, rows, C, C / E, rpw, 0.f};
  if (int rc = bind_window(a, win, rows, residual ? 7 : 3)) return rc;
  // a workgroup reads and writes rows of its own only while source and destination are in the same order
  TCH_CHECK_ARG(!(dx == dy && a.win_out != a.win_dy) && !(dx == residual && a.win_out != a.win_add),
                "layernorm_bwd: dx may overwrite an operand only where both are in the same order");
  const double bytes = static_cast<double>(rows) * C * (dtype == kBF16 ? 6.0 : 12.0);
  const LnShape sh = ln_shape(a.cc);
  int rc = dtype == kBF16 ? launch(ctx, ln_kernel_for<bf16, true>(sh), dim3(blocks), dim3(256), a, "ln_bwd_kernel<bf16>", bytes, 1)
                          : launch(ctx, ln_kernel_for<float, true>(sh), dim3(blocks), dim3(256), a, "ln_bwd_kernel<f32>", bytes, 1);
  if (rc) return rc;
  ColSumArgs s{partial, dgamma, dbeta, blocks, C, accumulate};
  return launch(ctx, col_sum_kernel, dim3((C + 7) / 8), dim3(256), s, "col_sum_kernel", 8.0 * blocks * C, 1);
}

int gelu_fwd(Context* ctx, int dtype, const void* x, void* y, int64_t n, int tanh_form) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "gelu_fwd: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(x && y && n > 0 && n % E == 0, "gelu_fwd: null tensor, or a size that is not a multiple of a 16-byte chunk");
  GeluArgs a{x, nullptr, y, n / E, tanh_form};
  const double bytes = static_cast<double>(n) * (dtype == kBF16 ? 4.0 : 8.0);
  const dim3 grid(flat_blocks(a.chunks));
  return dtype == kBF16 ? launch(ctx, gelu_kernel<bf16, 0>, grid, dim3(256), a, "gelu_kernel<bf16,fwd>", bytes, 1)
                        : launch(ctx, gelu_kernel<float, 0>, grid, dim3(256), a, "gelu_kernel<f32,fwd>", bytes, 1);
}

int gelu_bwd(Context* ctx, int dtype, const void* dy, const void* x, void* dx, int64_t n, int tanh_form) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "gelu_bwd: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(dy && x && dx && n > 0 && n % E == 0, "gelu_bwd: null tensor, or a size that is not a multiple of a 16-byte chunk");
  GeluArgs a{x, dy, dx, n / E, tanh_form};
  const double bytes = static_cast<double>(n) * (dtype == kBF16 ? 6.0 : 12.0);
  const dim3 grid(flat_blocks(a.chunks));
  return dtype == kBF16 ? launch(ctx, gelu_kernel<bf16, 1>, grid, dim3(256), a, "gelu_kernel<bf16,bwd>", bytes, 1)
                        : launch(ctx, gelu_kernel<float, 1>, grid, dim3(256), a, "gelu_kernel<f32,bwd>", bytes, 1);
}

int attn_softmax_fwd(Context* ctx, int dtype, const void* scores, void* probs, int64_t batch, int heads, int Lq, int Lk,
                     float scale, const float* bias, const float* mask, int windows, int causal) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "attn_softmax: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(scores && probs && batch > 0 && heads > 0 && Lq > 0 && Lk > 0, "attn_softmax_fwd: bad arguments");
  TCH_CHECK_ARG(!mask || (windows > 0 && batch % windows == 0), "attn_softmax_fwd: batch must be a multiple of the windows");
  TCH_CHECK_ARG(!causal || Lq == Lk, "attn_softmax_fwd: the causal form needs square score matrices");
  SoftmaxArgs a{scores, nullptr, probs, bias, mask, batch * heads * Lq, heads, Lq, Lk, mask ? windows : 1, causal, scale};
  const double bytes = static_cast<double>(a.rows) * Lk * (dtype == kBF16 ? 4.0 : 8.0);
  const dim3 grid(static_cast<unsigned>((a.rows + 3) / 4));
  return dtype == kBF16 ? launch(ctx, attn_softmax_kernel<bf16, 0>, grid, dim3(256), a, "attn_softmax_kernel<bf16,fwd>", bytes, 1)
                        : launch(ctx, attn_softmax_kernel<float, 0>, grid, dim3(256), a, "attn_softmax_kernel<f32,fwd>", bytes, 1);
}

int attn_softmax_bwd(Context* ctx, int dtype, const void* probs, const void* dprobs, void* dscores, int64_t rows, int Lq,
                     int Lk, float scale, int causal) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "attn_softmax: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(probs && dprobs && dscores && rows > 0 && Lk > 0 && Lq > 0 && rows % Lq == 0, "attn_softmax_bwd: bad arguments");
  TCH_CHECK_ARG(!causal || Lq == Lk, "attn_softmax_bwd: the causal form needs square score matrices");
  SoftmaxArgs a{probs, dprobs, dscores, nullptr, nullptr, rows, 1, Lq, Lk, 1, causal, scale};
  const double bytes = static_cast<double>(rows) * Lk * (dtype == kBF16 ? 6.0 : 12.0);
  const dim3 grid(static_cast<unsigned>((rows + 3) / 4));
  return dtype == kBF16 ? launch(ctx, attn_softmax_kernel<bf16, 1>, grid, dim3(256), a, "attn_softmax_kernel<bf16,bwd>", bytes, 1)
                        : launch(ctx, attn_softmax_kernel<float, 1>, grid, dim3(256), a, "attn_softmax_kernel<f32,bwd>", bytes, 1);
}

int adamw_step(Context* ctx, float* param, const float* grad, float* exp_avg, float* exp_avg_sq, void* shadow_bf16,
               int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay, int* step_dev,
               float* scalars_dev) {
  TCH_CHECK_ARG(param && grad && exp_avg && exp_avg_sq && step_dev && scalars_dev && n > 0, "adamw_step: null tensor or empty");
  AdamTickArgs t{step_dev, scalars_dev, beta1, beta2};
  if (int rc = launch(ctx, adamw_tick_kernel, dim3(1), dim3(64), t, "adamw_tick_kernel", 12.0, 1)) return rc;
  AdamArgs a{param,
             grad,
             exp_avg,
             exp_avg_sq,
             static_cast<uint16_t*>(shadow_bf16),
             scalars_dev,
             n,
             static_cast<float>(lr),
             static_cast<float>(beta2),
             static_cast<float>(1.0 - beta1),
             static_cast<float>(1.0 - beta2),
             static_cast<float>(eps),
             static_cast<float>(1.0 - lr * weight_decay),
             0};
  a.aligned = ((reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(grad) | reinterpret_cast<uintptr_t>(exp_avg) |
                reinterpret_cast<uintptr_t>(exp_avg_sq)) & 15) == 0 &&
              (reinterpret_cast<uintptr_t>(shadow_bf16) & 7) == 0;
  return launch(ctx, adamw_kernel, dim3(flat_blocks((n + 3) / 4)), dim3(256), a, "adamw_kernel",
                static_cast<double>(n) * (shadow_bf16 ? 30.0 : 28.0), 1);
}

int embedding_fwd(Context* ctx, int dtype, const int64_t* ids, const void* wte, const void* wpe, void* out, int B, int T,
                  int C, int vocab) {
  if (int rc = check_rows("embedding_fwd", dtype, static_cast<int64_t>(B) * T, C)) return rc;
  TCH_CHECK_ARG(ids && wte && wpe && out && vocab > 0, "embedding_fwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  EmbedArgs a{ids, wte, wpe, out, nullptr, nullptr, nullptr, static_cast<int64_t>(B) * T, T, C, C / E, vocab, B, 0, nullptr, nullptr};
  const double bytes = static_cast<double>(a.tokens) * C * (dtype == kBF16 ? 6.0 : 12.0);
  const dim3 grid(flat_blocks(a.tokens * a.cc));
  return dtype == kBF16 ? launch(ctx, embed_fwd_kernel<bf16>, grid, dim3(256), a, "embed_fwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, embed_fwd_kernel<float>, grid, dim3(256), a, "embed_fwd_kernel<f32>", bytes, 1);
}

int embedding_bwd(Context* ctx, int dtype, const int64_t* ids, const void* dy, float* dwte, float* dwpe, int B, int T,
                  int C, int vocab, int accumulate_wpe, int32_t* chain) {
  if (int rc = check_rows("embedding_bwd", dtype, static_cast<int64_t>(B) * T, C)) return rc;
  TCH_CHECK_ARG(ids && dy && dwte && dwpe && vocab > 0, "embedding_bwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  const int n = B * T;
  EmbedArgs a{ids, nullptr, nullptr, nullptr, dy, dwte, dwpe, static_cast<int64_t>(B) * T, T, C, C / E, vocab, B,
              accumulate_wpe, chain, chain ? chain + n : nullptr};
  if (chain) {
    ChainArgs ca{ids, chain, chain + n, n, vocab};
    if (int rc = launch(ctx, embed_chain_kernel, dim3((n + 63) / 64), dim3(256), ca, "embed_chain_kernel", 16.0 * n, 1))
      return rc;
  }
  const double bytes = static_cast<double>(a.tokens) * C * (dtype == kBF16 ? 2.0 : 4.0) + 8.0 * a.tokens * C;
  const dim3 grid(flat_blocks(a.tokens * a.cc));
  return dtype == kBF16 ? launch(ctx, embed_bwd_kernel<bf16>, grid, dim3(256), a, "embed_bwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, embed_bwd_kernel<float>, grid, dim3(256), a, "embed_bwd_kernel<f32>", bytes, 1);
}

}  // namespace tch
