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

// The same for at most one chunk of channels per pixel (images: 3 -> one 16-byte chunk): a thread makes one
// pixel, reads its channels from the planes (neighbouring threads read neighbouring addresses of each plane)
// and stores the chunk at once.
template <typename T>
__global__ __launch_bounds__(256) void nchw_to_nhwc_chunk_kernel(NchwArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t pix = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t plane = static_cast<int64_t>(p.H) * p.W;
  if (pix >= p.N * plane) return;
  const int64_t n = pix / plane, hw = pix - n * plane;
  float v[E];
#pragma unroll
  for (int c = 0; c < E; ++c) v[c] = c < p.C ? p.x[(n * p.C + c) * plane + hw] : 0.f;
  static_cast<uint4*>(p.y)[pix] = float_to_chunk<T>(v).u;
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

// [K][R*S][C] -> [C][R*S][K] for a whole table of filters in ONE launch: the data-gradient
// GEMM wants the filter with the output channel as its contiguous (reduction) dimension.
// One workgroup moves one 32x32 (k, c) tile of one tap through LDS so that both the read
// (along c) and the write (along k) are coalesced.
struct TransposeArgs {
  const void* src;
  void* dst;
  const int64_t* table;  // per filter: first tile, element offset, K, RS, C
  int n_filters;
};

template <typename T>
__global__ __launch_bounds__(256) void filter_transpose_kernel(TransposeArgs p) {
  __shared__ T tile[32][33];
  const int64_t bid = blockIdx.x;
  int lo = 0, hi = p.n_filters - 1;
  while (lo < hi) {  // last filter whose first tile is <= bid
    int mid = (lo + hi + 1) >> 1;
    if (p.table[mid * 5] <= bid) lo = mid; else hi = mid - 1;
  }
  const int64_t* e = p.table + lo * 5;
  const int64_t off = e[1];
  const int K = static_cast<int>(e[2]), RS = static_cast<int>(e[3]), C = static_cast<int>(e[4]);
  const int tiles_c = (C + 31) / 32, tiles_k = (K + 31) / 32;
  int64_t t = bid - e[0];
  const int tc = static_cast<int>(t % tiles_c);
  t /= tiles_c;
  const int tk = static_cast<int>(t % tiles_k);
  const int rs = static_cast<int>(t / tiles_k);
  const T* src = static_cast<const T*>(p.src) + off;
  T* dst = static_cast<T*>(p.dst) + off;
  // 16-byte accesses where the filter allows them (K, C and the offset multiples of a chunk): a thread moves one
  // chunk of a tile row in, one chunk of a transposed row out; element by element otherwise
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int TPR = 32 / E;   // threads per tile row
  if (K % E == 0 && C % E == 0 && off % E == 0) {
    const int row = threadIdx.x / TPR, seg = threadIdx.x % TPR;
    if (threadIdx.x < 32 * TPR) {
      const int k = tk * 32 + row, c = tc * 32 + seg * E;
      if (k < K && c < C) {
        union { uint4 u; T e[E]; } v;
        v.u = *reinterpret_cast<const uint4*>(src + (static_cast<int64_t>(k) * RS + rs) * C + c);
#pragma unroll
        for (int e = 0; e < E; ++e) tile[row][seg * E + e] = v.e[e];
      }
    }
    __syncthreads();
    if (threadIdx.x < 32 * TPR) {
      const int c = tc * 32 + row, k = tk * 32 + seg * E;
      if (c < C && k < K) {
        union { uint4 u; T e[E]; } v;
#pragma unroll
        for (int e = 0; e < E; ++e) v.e[e] = tile[seg * E + e][row];
        *reinterpret_cast<uint4*>(dst + (static_cast<int64_t>(c) * RS + rs) * K + k) = v.u;
      }
    }
    return;
  }
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = tk * 32 + ty + i * 8, c = tc * 32 + tx;
    if (k < K && c < C) tile[ty + i * 8][tx] = src[(static_cast<int64_t>(k) * RS + rs) * C + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tc * 32 + ty + i * 8, k = tk * 32 + tx;
    if (k < K && c < C) dst[(static_cast<int64_t>(c) * RS + rs) * K + k] = tile[tx][ty + i * 8];
  }
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
  const double bytes = static_cast<double>(N) * H * W * (C * 4.0 + Cpad * (dtype == kBF16 ? 2.0 : 4.0));
  if (Cpad == (dtype == kBF16 ? 8 : 4)) {
    const dim3 pixels(static_cast<unsigned>((static_cast<int64_t>(N) * H * W + 255) / 256));
    return dtype == kBF16 ? launch(ctx, nchw_to_nhwc_chunk_kernel<bf16>, pixels, dim3(256), a, "nchw_to_nhwc_kernel<bf16>", bytes, 1)
                          : launch(ctx, nchw_to_nhwc_chunk_kernel<float>, pixels, dim3(256), a, "nchw_to_nhwc_kernel<f32>", bytes, 1);
  }
  return dtype == kBF16 ? launch(ctx, nchw_to_nhwc_kernel<bf16>, grid, dim3(256), a, "nchw_to_nhwc_kernel<bf16>", bytes, 1)
                        : launch(ctx, nchw_to_nhwc_kernel<float>, grid, dim3(256), a, "nchw_to_nhwc_kernel<f32>", bytes, 1);
}

int cast_f32(Context* ctx, int dtype, const float* src, void* dst, int64_t n) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "cast_f32: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(src && dst && n > 0, "cast_f32: bad arguments");
  CastArgs a{src, dst, n};
  return dtype == kBF16 ? launch(ctx, cast_from_f32_kernel<bf16>, dim3(blocks_for(n)), dim3(256), a, "cast_from_f32_kernel", 6.0 * n, 1)
                        : launch(ctx, cast_from_f32_kernel<float>, dim3(blocks_for(n)), dim3(256), a, "cast_from_f32_kernel", 8.0 * n, 1);
}

int cast_to_f32(Context* ctx, int dtype, const void* src, float* dst, int64_t n) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "cast_to_f32: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(src && dst && n > 0, "cast_to_f32: bad arguments");
  CastArgs a{src, dst, n};
  return dtype == kBF16 ? launch(ctx, cast_to_f32_kernel<bf16>, dim3(blocks_for(n)), dim3(256), a, "cast_to_f32_kernel", 6.0 * n, 1)
                        : launch(ctx, cast_to_f32_kernel<float>, dim3(blocks_for(n)), dim3(256), a, "cast_to_f32_kernel", 8.0 * n, 1);
}

}  // namespace tch

namespace tch {

int filter_transpose_batched(Context* ctx, int dtype, const void* src, void* dst, const int64_t* table_dev,
                             int n_filters, int64_t total_tiles, int64_t total_elems) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "filter_transpose: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(src && dst && table_dev && n_filters > 0, "filter_transpose: bad arguments");
  TCH_CHECK_ARG(total_tiles > 0 && total_tiles < (1ll << 31), "filter_transpose: tile count out of range");
  TransposeArgs a{src, dst, table_dev, n_filters};
  const double bytes = 2.0 * total_elems * (dtype == kBF16 ? 2.0 : 4.0);
  dim3 grid(static_cast<unsigned>(total_tiles));
  return dtype == kBF16 ? launch(ctx, filter_transpose_kernel<bf16>, grid, dim3(256), a, "filter_transpose_kernel<bf16>", bytes, 1)
                        : launch(ctx, filter_transpose_kernel<float>, grid, dim3(256), a, "filter_transpose_kernel<f32>", bytes, 1);
}

}  // namespace tch
