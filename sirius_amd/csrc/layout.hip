// Layout and precision conversions at the edges of the step: the training
// scripts hand over NCHW fp32 images (reference: torch.randn batches built in
// pytorch/torch_col/dynamic_batch.py:394-410), the kernels work on NHWC with
// the channel count padded to a 16-byte chunk.
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

struct NchwArgs {
  const float* x;
  void* y;
  int N, C, H, W, Cpad;
  int64_t total;  // N*H*W*Cpad
};

template <typename T>
__global__ __launch_bounds__(256) void nchw_to_nhwc_kernel(NchwArgs p) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= p.total) return;
  const int c = static_cast<int>(i % p.Cpad);
  int64_t pix = i / p.Cpad;
  const int64_t hw = pix % (static_cast<int64_t>(p.H) * p.W);
  const int64_t n = pix / (static_cast<int64_t>(p.H) * p.W);
  float v = 0.f;
  if (c < p.C) v = p.x[(n * p.C + c) * p.H * p.W + hw];
  Elem<T>::store(static_cast<T*>(p.y) + i, v);
}

struct CastArgs {
  const void* src;
  void* dst;
  int64_t n;
};

template <typename T>
__global__ __launch_bounds__(256) void cast_from_f32_kernel(CastArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < p.n; i += stride)
    Elem<T>::store(static_cast<T*>(p.dst) + i, static_cast<const float*>(p.src)[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void cast_to_f32_kernel(CastArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < p.n; i += stride)
    static_cast<float*>(p.dst)[i] = Elem<T>::load(static_cast<const T*>(p.src) + i);
}

unsigned blocks_for(int64_t n) {
  int64_t b = (n + 255) / 256;
  if (b > 16384) b = 16384;
  if (b < 1) b = 1;
  return static_cast<unsigned>(b);
}

}  // namespace

int nchw_to_nhwc_pad(Context* ctx, int dtype, const float* x_nchw, void* y_nhwc, int N, int C, int H, int W, int Cpad) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "nchw_to_nhwc_pad: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(x_nchw && y_nhwc && N > 0 && C > 0 && H > 0 && W > 0 && Cpad >= C, "nchw_to_nhwc_pad: bad arguments");
  NchwArgs a{x_nchw, y_nhwc, N, C, H, W, Cpad, static_cast<int64_t>(N) * H * W * Cpad};
  dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
  return dtype == kBF16 ? launch(ctx, nchw_to_nhwc_kernel<bf16>, grid, dim3(256), a)
                        : launch(ctx, nchw_to_nhwc_kernel<float>, grid, dim3(256), a);
}

int cast_f32(Context* ctx, int dtype, const float* src, void* dst, int64_t n) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "cast_f32: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(src && dst && n > 0, "cast_f32: bad arguments");
  CastArgs a{src, dst, n};
  return dtype == kBF16 ? launch(ctx, cast_from_f32_kernel<bf16>, dim3(blocks_for(n)), dim3(256), a)
                        : launch(ctx, cast_from_f32_kernel<float>, dim3(blocks_for(n)), dim3(256), a);
}

int cast_to_f32(Context* ctx, int dtype, const void* src, float* dst, int64_t n) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "cast_to_f32: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(src && dst && n > 0, "cast_to_f32: bad arguments");
  CastArgs a{src, dst, n};
  return dtype == kBF16 ? launch(ctx, cast_to_f32_kernel<bf16>, dim3(blocks_for(n)), dim3(256), a)
                        : launch(ctx, cast_to_f32_kernel<float>, dim3(blocks_for(n)), dim3(256), a);
}

}  // namespace tch
