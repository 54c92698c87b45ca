// Max pooling (with argmax) and global average pooling over NHWC activations.
// HBM-bound: one lane per 16-byte chunk of channels.
//
// Arithmetic restated from torch.nn.MaxPool2d / AdaptiveAvgPool2d as used by
// torchvision's ResNet (reference call site train/resnet152.py:22).  Argmax
// tie rule of the CPU kernel: the window is scanned row-major, a later element
// replaces the current one only if it is strictly greater or NaN, so the FIRST
// maximum wins; the index is h*W + w inside the input plane.
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

struct MaxPoolArgs {
  const void* x;
  void* y;
  int32_t* index;
  int N, H, W, C, Ho, Wo, cc;
  int ksize, stride, pad;
  int64_t total;  // output chunks (fwd) or input chunks (bwd)
};

template <typename T>
__global__ __launch_bounds__(256) void maxpool_fwd_kernel(MaxPoolArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= p.total) return;
  const int col = static_cast<int>(i % p.cc);
  int64_t pix = i / p.cc;
  const int ow = static_cast<int>(pix % p.Wo);
  pix /= p.Wo;
  const int oh = static_cast<int>(pix % p.Ho);
  const int n = static_cast<int>(pix / p.Ho);
  int h0 = oh * p.stride - p.pad, w0 = ow * p.stride - p.pad;
  int h1 = h0 + p.ksize, w1 = w0 + p.ksize;
  if (h1 > p.H) h1 = p.H;
  if (w1 > p.W) w1 = p.W;
  if (h0 < 0) h0 = 0;
  if (w0 < 0) w0 = 0;
  float best[E];
  int32_t arg[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    best[e] = -INFINITY;
    arg[e] = h0 * p.W + w0;
  }
  const uint4* src = static_cast<const uint4*>(p.x);
  for (int h = h0; h < h1; ++h) {
    for (int w = w0; w < w1; ++w) {
      Chunk c;
      c.u = src[(static_cast<int64_t>(n) * p.H * p.W + h * p.W + w) * p.cc + col];
      float v[E];
      chunk_to_float<T>(c, v);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (v[e] > best[e] || v[e] != v[e]) {
          best[e] = v[e];
          arg[e] = h * p.W + w;
        }
      }
    }
  }
  static_cast<uint4*>(p.y)[i] = float_to_chunk<T>(best).u;
  int32_t* dst = p.index + i * E;
#pragma unroll
  for (int e = 0; e < E; e += 4) *reinterpret_cast<int4*>(dst + e) = make_int4(arg[e], arg[e + 1], arg[e + 2], arg[e + 3]);
}

// Gather form: every input pixel looks at the (at most ceil(k/s)^2) windows
// that cover it and takes the gradient of those that chose it.  Deterministic,
// no atomics.
template <typename T>
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(MaxPoolArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= p.total) return;
  const int col = static_cast<int>(i % p.cc);
  int64_t pix = i / p.cc;
  const int w = static_cast<int>(pix % p.W);
  pix /= p.W;
  const int h = static_cast<int>(pix % p.H);
  const int n = static_cast<int>(pix / p.H);
  const int self = h * p.W + w;
  // windows oh with oh*stride - pad <= h < oh*stride - pad + ksize
  int oh_hi = (h + p.pad) / p.stride;
  int ow_hi = (w + p.pad) / p.stride;
  int oh_lo = (h + p.pad - p.ksize + p.stride) / p.stride;  // ceil((h+pad-k+1)/stride)
  int ow_lo = (w + p.pad - p.ksize + p.stride) / p.stride;
  if (h + p.pad - p.ksize + 1 <= 0) oh_lo = 0;
  if (w + p.pad - p.ksize + 1 <= 0) ow_lo = 0;
  if (oh_hi >= p.Ho) oh_hi = p.Ho - 1;
  if (ow_hi >= p.Wo) ow_hi = p.Wo - 1;
  float g[E];
#pragma unroll
  for (int e = 0; e < E; ++e) g[e] = 0.f;
  const uint4* dy = static_cast<const uint4*>(p.x);
  for (int oh = oh_lo; oh <= oh_hi; ++oh) {
    for (int ow = ow_lo; ow <= ow_hi; ++ow) {
      const int64_t o = (static_cast<int64_t>(n) * p.Ho * p.Wo + oh * p.Wo + ow) * p.cc + col;
      const int32_t* idx = p.index + o * E;
      Chunk c;
      c.u = dy[o];
      float v[E];
      chunk_to_float<T>(c, v);
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (idx[e] == self) g[e] += v[e];
    }
  }
  static_cast<uint4*>(p.y)[i] = float_to_chunk<T>(g).u;
}

struct AvgPoolArgs {
  const void* x;
  void* y;
  int N, HW, cc;
  float inv;
  int64_t total;
};

template <typename T>
__global__ __launch_bounds__(256) void avgpool_fwd_kernel(AvgPoolArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= p.total) return;
  const int col = static_cast<int>(i % p.cc);
  const int64_t n = i / p.cc;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = 0.f;
  const uint4* src = static_cast<const uint4*>(p.x) + n * p.HW * p.cc + col;
  for (int j = 0; j < p.HW; ++j) {
    Chunk c;
    c.u = src[static_cast<int64_t>(j) * p.cc];
    float v[E];
    chunk_to_float<T>(c, v);
#pragma unroll
    for (int e = 0; e < E; ++e) s[e] += v[e];
  }
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] *= p.inv;
  static_cast<uint4*>(p.y)[i] = float_to_chunk<T>(s).u;
}

template <typename T>
__global__ __launch_bounds__(256) void avgpool_bwd_kernel(AvgPoolArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // input chunk
  if (i >= p.total) return;
  const int col = static_cast<int>(i % p.cc);
  const int64_t n = i / (static_cast<int64_t>(p.cc) * p.HW);
  Chunk c;
  c.u = static_cast<const uint4*>(p.x)[n * p.cc + col];
  float v[E];
  chunk_to_float<T>(c, v);
#pragma unroll
  for (int e = 0; e < E; ++e) v[e] *= p.inv;
  static_cast<uint4*>(p.y)[i] = float_to_chunk<T>(v).u;
}

int pool_check(int dtype, int N, int H, int W, int C, int ksize, int stride, int pad) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "pool: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(N > 0 && H > 0 && W > 0 && C > 0 && C % E == 0, "pool: C must be a positive multiple of a 16-byte chunk");
  TCH_CHECK_ARG(ksize > 0 && stride > 0 && pad >= 0 && pad * 2 <= ksize, "pool: bad window");
  TCH_CHECK_ARG(static_cast<int64_t>(H) * W < (1ll << 31), "pool: plane too large for int32 indices");
  return 0;
}

}  // namespace

int maxpool_fwd(Context* ctx, int dtype, const void* x, void* y, int32_t* index, int N, int H, int W, int C, int ksize,
                int stride, int pad) {
  if (int rc = pool_check(dtype, N, H, W, C, ksize, stride, pad)) return rc;
  TCH_CHECK_ARG(x && y && index, "maxpool_fwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  MaxPoolArgs a{x, y, index, N, H, W, C, (H + 2 * pad - ksize) / stride + 1, (W + 2 * pad - ksize) / stride + 1, C / E,
                ksize, stride, pad, 0};
  TCH_CHECK_ARG(a.Ho > 0 && a.Wo > 0, "maxpool_fwd: empty output");
  a.total = static_cast<int64_t>(N) * a.Ho * a.Wo * a.cc;
  dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double bytes = static_cast<double>(N) * C * (H * W * eb + a.Ho * a.Wo * (eb + 4.0));
  return dtype == kBF16 ? launch(ctx, maxpool_fwd_kernel<bf16>, grid, dim3(256), a, "maxpool_fwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, maxpool_fwd_kernel<float>, grid, dim3(256), a, "maxpool_fwd_kernel<f32>", bytes, 1);
}

int maxpool_bwd(Context* ctx, int dtype, const void* dy, const int32_t* index, void* dx, int N, int H, int W, int C,
                int ksize, int stride, int pad) {
  if (int rc = pool_check(dtype, N, H, W, C, ksize, stride, pad)) return rc;
  TCH_CHECK_ARG(dy && dx && index, "maxpool_bwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  MaxPoolArgs a{dy, dx, const_cast<int32_t*>(index), N, H, W, C, (H + 2 * pad - ksize) / stride + 1,
                (W + 2 * pad - ksize) / stride + 1, C / E, ksize, stride, pad, 0};
  a.total = static_cast<int64_t>(N) * H * W * a.cc;
  dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
  const double eb = dtype == kBF16 ? 2.0 : 4.0;
  const double bytes = static_cast<double>(N) * C * (H * W * eb + a.Ho * a.Wo * (eb + 4.0));
  return dtype == kBF16 ? launch(ctx, maxpool_bwd_kernel<bf16>, grid, dim3(256), a, "maxpool_bwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, maxpool_bwd_kernel<float>, grid, dim3(256), a, "maxpool_bwd_kernel<f32>", bytes, 1);
}

int avgpool_fwd(Context* ctx, int dtype, const void* x, void* y, int N, int HW, int C) {
  if (int rc = pool_check(dtype, N, HW, 1, C, 1, 1, 0)) return rc;
  TCH_CHECK_ARG(x && y, "avgpool_fwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  AvgPoolArgs a{x, y, N, HW, C / E, 1.0f / static_cast<float>(HW), static_cast<int64_t>(N) * (C / E)};
  dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
  const double bytes = static_cast<double>(N) * C * (HW + 1) * (dtype == kBF16 ? 2.0 : 4.0);
  return dtype == kBF16 ? launch(ctx, avgpool_fwd_kernel<bf16>, grid, dim3(256), a, "avgpool_fwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, avgpool_fwd_kernel<float>, grid, dim3(256), a, "avgpool_fwd_kernel<f32>", bytes, 1);
}

int avgpool_bwd(Context* ctx, int dtype, const void* dy, void* dx, int N, int HW, int C) {
  if (int rc = pool_check(dtype, N, HW, 1, C, 1, 1, 0)) return rc;
  TCH_CHECK_ARG(dy && dx, "avgpool_bwd: null tensor");
  const int E = dtype == kBF16 ? 8 : 4;
  AvgPoolArgs a{dy, dx, N, HW, C / E, 1.0f / static_cast<float>(HW), static_cast<int64_t>(N) * HW * (C / E)};
  dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
  const double bytes = static_cast<double>(N) * C * (HW + 1) * (dtype == kBF16 ? 2.0 : 4.0);
  return dtype == kBF16 ? launch(ctx, avgpool_bwd_kernel<bf16>, grid, dim3(256), a, "avgpool_bwd_kernel<bf16>", bytes, 1)
                        : launch(ctx, avgpool_bwd_kernel<float>, grid, dim3(256), a, "avgpool_bwd_kernel<f32>", bytes, 1);
}

}  // namespace tch
