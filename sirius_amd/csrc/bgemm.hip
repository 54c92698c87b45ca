// Batched, strided GEMM on MFMA for the attention products of the transformer steps:
//   C[z](m, n) (+)= alpha * sum_k A[z](m, k) * B[z](n, k)
// A(m, k) sits at a + z-offset + m * a_rs + k * a_cs, B(n, k) at b + z-offset + n * b_rs + k * b_cs;
// for each operand one of the two strides is 1 (the contiguous one), so the same kernel covers
//   Q K^T        (both k-contiguous)            scores
//   P V          (A k-contiguous, B n-contiguous)
//   P^T dO, dS^T Q   (A m-contiguous, B n-contiguous)   dV, dK
//   dO V^T, dS K     (k-contiguous / n-contiguous)      dP, dQ
// without transposed copies.  A batch index z splits into (z / inner, z % inner) with separate
// offsets, which addresses head h of sample b inside a packed [B, T, 3C] projection.
//
// Tile 64 x 64 x 32, four wavefronts of 32 x 32 (one mfma 32x32 accumulator each).  Operands go
// global -> registers -> LDS in the [row][k] layout the MFMA fragments read; a chunk that is not
// contiguous along k is scattered element by element on its way into LDS.
//
// Reference call sites of the products: window attention q @ k^T and attn @ v
// (train/swin_b_tiny.py:94-110); GPT-2 attention inside transformers (train/gpt2.py:26).
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

constexpr int kTile = 64;
constexpr int kBK = 32;

struct BgemmArgs {
  const void* a;
  const void* b;
  void* c;
  int M, N, K;
  int64_t a_rs, a_cs, b_rs, b_cs, ldc;
  int batch_inner;
  int64_t a_bo, a_bi, b_bo, b_bi, c_bo, c_bi;  // offsets per outer / inner batch index, in elements
  float alpha;
  int accumulate;
  int tiles_m, tiles_n;
};

template <typename T>
__device__ inline void mma_step(const Chunk& first, const Chunk& second, f32x16_t& acc);
template <>
__device__ inline void mma_step<bf16>(const Chunk& first, const Chunk& second, f32x16_t& acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(first.h, second.h, acc, 0, 0, 0);
}
template <>
__device__ inline void mma_step<float>(const Chunk& first, const Chunk& second, f32x16_t& acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(first.f[e], second.f[e], acc, 0, 0, 0);
}

// One operand tile [64 rows][kBK] into LDS rows of (kBK / E + 1) chunks.  `rows`/`ks` are what is
// left of the matrix from this tile's origin; everything beyond reads as zero.
template <typename T>
__device__ inline void stage_tile(const T* base, int64_t rs, int64_t cs, int rows, int ks, unsigned char* lds, int tid) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int KCH = kBK / E;                    // chunks along k per row
  constexpr int ROW_BYTES = (KCH + 1) * 16;
  constexpr int CHUNKS = kTile * kBK / E;          // per tile
  constexpr int PER_THREAD = CHUNKS / 256;
  static_assert(CHUNKS % 256 == 0, "tile/loader mismatch");
#pragma unroll
  for (int it = 0; it < PER_THREAD; ++it) {
    const int q = tid + it * 256;
    if (cs == 1) {
      // chunk = E consecutive k of one row
      const int r = q / KCH, kc = (q - r * KCH) * E;
      const T* src = base + static_cast<int64_t>(r) * rs + kc;
      Chunk ch = zero_chunk();
      if (r < rows) {
        if (kc + E <= ks && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
          ch.u = *reinterpret_cast<const uint4*>(src);
        } else {
          T* dst = reinterpret_cast<T*>(&ch);
#pragma unroll
          for (int e = 0; e < E; ++e)
            if (kc + e < ks) dst[e] = src[e];
        }
      }
      *reinterpret_cast<uint4*>(lds + r * ROW_BYTES + kc * sizeof(T)) = ch.u;
    } else {
      // chunk = E consecutive rows at one k (rs == 1)
      constexpr int RCH = kTile / E;
      const int k = q / RCH, r0 = (q - k * RCH) * E;
      const T* src = base + static_cast<int64_t>(k) * cs + r0;
      Chunk ch = zero_chunk();
      if (k < ks) {
        if (r0 + E <= rows && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
          ch.u = *reinterpret_cast<const uint4*>(src);
        } else {
          T* dst = reinterpret_cast<T*>(&ch);
#pragma unroll
          for (int e = 0; e < E; ++e)
            if (r0 + e < rows) dst[e] = src[e];
        }
      }
      const T* vals = reinterpret_cast<const T*>(&ch);
#pragma unroll
      for (int e = 0; e < E; ++e) *reinterpret_cast<T*>(lds + (r0 + e) * ROW_BYTES + k * sizeof(T)) = vals[e];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bgemm_kernel(BgemmArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int KCH = kBK / E;
  constexpr int ROW_BYTES = (KCH + 1) * 16;
  constexpr int TILE_BYTES = kTile * ROW_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * TILE_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tile = blockIdx.x;
  const int tile_m = tile / p.tiles_n, tile_n = tile - tile_m * p.tiles_n;
  const int m0 = tile_m * kTile, n0 = tile_n * kTile;
  const int z = blockIdx.y;
  const int zo = z / p.batch_inner, zi = z - zo * p.batch_inner;
  const T* A = static_cast<const T*>(p.a) + zo * p.a_bo + zi * p.a_bi + static_cast<int64_t>(m0) * p.a_rs;
  const T* B = static_cast<const T*>(p.b) + zo * p.b_bo + zi * p.b_bi + static_cast<int64_t>(n0) * p.b_rs;

  f32x16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  const int frag_row = lane & 31, frag_half = lane >> 5;
  for (int k0 = 0; k0 < p.K; k0 += kBK) {
    __syncthreads();
    stage_tile<T>(A + static_cast<int64_t>(k0) * p.a_cs, p.a_rs, p.a_cs, p.M - m0, p.K - k0, lds, tid);
    stage_tile<T>(B + static_cast<int64_t>(k0) * p.b_cs, p.b_rs, p.b_cs, p.N - n0, p.K - k0, lds + TILE_BYTES, tid);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KCH / 2; ++kk) {
      Chunk fa, fb;
      fa.u = *reinterpret_cast<const uint4*>(lds + (wm * 32 + frag_row) * ROW_BYTES + (kk * 2 + frag_half) * 16);
      fb.u = *reinterpret_cast<const uint4*>(lds + TILE_BYTES + (wn * 32 + frag_row) * ROW_BYTES + (kk * 2 + frag_half) * 16);
      mma_step<T>(fb, fa, acc);  // B rows -> accumulator registers, A rows -> lanes
    }
  }
  // lane (l & 31) holds row m; register 4 j + i holds column 8 j + 4 (l >> 5) + i
  const int m = m0 + wm * 32 + frag_row;
  if (m >= p.M) return;
  T* Crow = static_cast<T*>(p.c) + zo * p.c_bo + zi * p.c_bi + static_cast<int64_t>(m) * p.ldc;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + wn * 32 + 8 * j + 4 * frag_half + i;
      if (n < p.N) {
        float v = p.alpha * acc[4 * j + i];
        if (p.accumulate) v += Elem<T>::load(Crow + n);
        Elem<T>::store(Crow + n, v);
      }
    }
  }
}

}  // namespace

int batched_gemm(Context* ctx, int dtype, const void* a, const void* b, void* c, int M, int N, int K, int64_t a_rs,
                 int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t ldc, int batch_outer, int batch_inner, int64_t a_bo,
                 int64_t a_bi, int64_t b_bo, int64_t b_bi, int64_t c_bo, int64_t c_bi, float alpha, int accumulate) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "batched_gemm: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(a && b && c && M > 0 && N > 0 && K > 0, "batched_gemm: null tensor or empty shape");
  TCH_CHECK_ARG(batch_outer > 0 && batch_inner > 0 && static_cast<int64_t>(batch_outer) * batch_inner <= 65535,
                "batched_gemm: batch count must be in [1, 65535]");
  TCH_CHECK_ARG((a_rs == 1 || a_cs == 1) && (b_rs == 1 || b_cs == 1), "batched_gemm: one stride of each operand must be 1");
  TCH_CHECK_ARG(a_rs > 0 && a_cs > 0 && b_rs > 0 && b_cs > 0 && ldc >= N, "batched_gemm: bad strides");
  BgemmArgs g{a, b, c, M, N, K, a_rs, a_cs, b_rs, b_cs, ldc, batch_inner, a_bo, a_bi, b_bo, b_bi, c_bo, c_bi, alpha,
              accumulate, (M + kTile - 1) / kTile, (N + kTile - 1) / kTile};
  const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  TCH_CHECK_ARG(tiles <= 0x7fffffff, "batched_gemm: grid out of range");
  const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(batch_outer * batch_inner));
  const double flops = 2.0 * M * N * static_cast<double>(K) * batch_outer * batch_inner;
  return dtype == kBF16 ? launch(ctx, bgemm_kernel<bf16>, grid, dim3(256), g, "bgemm_kernel<bf16>", flops, 0)
                        : launch(ctx, bgemm_kernel<float>, grid, dim3(256), g, "bgemm_kernel<f32>", flops, 0);
}

}  // namespace tch
