// Batched, strided GEMM on MFMA for the attention products of the transformer steps:
//   C[z](m, n) (+)= alpha * sum_k A[z](m, k) * B[z](n, k)
// A(m, k) sits at a + z-offset + m * a_rs + k * a_cs, B(n, k) at b + z-offset + n * b_rs + k * b_cs;
// for each operand one of the two strides is 1 (the contiguous one), so the same kernel covers
//   Q K^T        (both k-contiguous)            scores
//   P V          (A k-contiguous, B n-contiguous)
//   P^T dO, dS^T Q   (A m-contiguous, B n-contiguous)   dV, dK
//   dO V^T, dS K     (k-contiguous / n-contiguous)      dP, dQ
// without transposed copies.  `causal` names what a causal mask leaves of a square problem, so that
// the other half is neither computed nor read:
//   1  only C(m, n) with n <= m is wanted: tiles wholly above the diagonal are left unwritten
//   2  A(m, k) is zero for k > m: the reduction stops at the tile's last row       (P V, dS K)
//   3  A(m, k) is zero for k < m: the reduction starts at the tile's first row     (P^T dO, dS^T Q)
// A batch index z splits into (z / inner, z % inner) with separate
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
  int causal;
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
  constexpr int STAGE_LD = kTile + 4;  // floats per row of the output staging tile
  constexpr int STAGE_BYTES = kTile * STAGE_LD * 4;
  constexpr int LDS_BYTES = 2 * TILE_BYTES > STAGE_BYTES ? 2 * TILE_BYTES : STAGE_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tile = blockIdx.x;
  const int tile_m = tile / p.tiles_n, tile_n = tile - tile_m * p.tiles_n;
  const int m0 = tile_m * kTile, n0 = tile_n * kTile;
  if (p.causal == 1 && n0 > m0 + kTile - 1) return;
  const int k_begin = p.causal == 3 ? (m0 / kBK) * kBK : 0;
  const int k_end = p.causal == 2 ? (m0 + kTile < p.K ? m0 + kTile : p.K) : p.K;
  const int z = blockIdx.y;
  const int zo = z / p.batch_inner, zi = z - zo * p.batch_inner;
  const T* A = static_cast<const T*>(p.a) + zo * p.a_bo + zi * p.a_bi + static_cast<int64_t>(m0) * p.a_rs;
  const T* B = static_cast<const T*>(p.b) + zo * p.b_bo + zi * p.b_bi + static_cast<int64_t>(n0) * p.b_rs;

  f32x16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  const int frag_row = lane & 31, frag_half = lane >> 5;
  for (int k0 = k_begin; k0 < k_end; k0 += kBK) {
    __syncthreads();
    stage_tile<T>(A + static_cast<int64_t>(k0) * p.a_cs, p.a_rs, p.a_cs, p.M - m0, k_end - k0, lds, tid);
    stage_tile<T>(B + static_cast<int64_t>(k0) * p.b_cs, p.b_rs, p.b_cs, p.N - n0, k_end - k0, lds + TILE_BYTES, tid);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KCH / 2; ++kk) {
      Chunk fa, fb;
      fa.u = *reinterpret_cast<const uint4*>(lds + (wm * 32 + frag_row) * ROW_BYTES + (kk * 2 + frag_half) * 16);
      fb.u = *reinterpret_cast<const uint4*>(lds + TILE_BYTES + (wn * 32 + frag_row) * ROW_BYTES + (kk * 2 + frag_half) * 16);
      mma_step<T>(fb, fa, acc);  // B rows -> accumulator registers, A rows -> lanes
    }
  }
  // lane (l & 31) holds row m; register 4 j + i holds column 8 j + 4 (l >> 5) + i.  The tile goes through
  // LDS so that every lane then owns E consecutive columns of one row: 16-byte stores along the rows of C.
  __syncthreads();
  float* stage = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int j = 0; j < 4; ++j)
    *reinterpret_cast<float4*>(stage + (wm * 32 + frag_row) * STAGE_LD + wn * 32 + 8 * j + 4 * frag_half) =
        make_float4(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]);
  __syncthreads();
  T* Ctile = static_cast<T*>(p.c) + zo * p.c_bo + zi * p.c_bi + static_cast<int64_t>(m0) * p.ldc + n0;
  const bool vector_ok = (p.ldc % E == 0) && ((reinterpret_cast<uintptr_t>(Ctile) & 15) == 0);
  constexpr int CH = kTile / E;
#pragma unroll
  for (int it = 0; it < kTile * CH / 256; ++it) {
    const int q = tid + it * 256;
    const int r = q / CH, c0 = (q - r * CH) * E;
    if (m0 + r >= p.M || n0 + c0 >= p.N) continue;
    float v[E];
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = p.alpha * stage[r * STAGE_LD + c0 + e];
    T* dst = Ctile + static_cast<int64_t>(r) * p.ldc + c0;
    if (vector_ok && n0 + c0 + E <= p.N) {
      if (p.accumulate) {
        Chunk old;
        old.u = *reinterpret_cast<const uint4*>(dst);
        float o[E];
        chunk_to_float<T>(old, o);
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] += o[e];
      }
      *reinterpret_cast<uint4*>(dst) = float_to_chunk<T>(v).u;
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (n0 + c0 + e < p.N) Elem<T>::store(dst + e, p.accumulate ? v[e] + Elem<T>::load(dst + e) : v[e]);
    }
  }
}

}  // namespace

int batched_gemm(Context* ctx, int dtype, const void* a, const void* b, void* c, int M, int N, int K, int64_t a_rs,
                 int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t ldc, int batch_outer, int batch_inner, int64_t a_bo,
                 int64_t a_bi, int64_t b_bo, int64_t b_bi, int64_t c_bo, int64_t c_bi, float alpha, int accumulate,
                 int causal) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "batched_gemm: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(a && b && c && M > 0 && N > 0 && K > 0, "batched_gemm: null tensor or empty shape");
  TCH_CHECK_ARG(batch_outer > 0 && batch_inner > 0 && static_cast<int64_t>(batch_outer) * batch_inner <= 65535,
                "batched_gemm: batch count must be in [1, 65535]");
  TCH_CHECK_ARG((a_rs == 1 || a_cs == 1) && (b_rs == 1 || b_cs == 1), "batched_gemm: one stride of each operand must be 1");
  TCH_CHECK_ARG(a_rs > 0 && a_cs > 0 && b_rs > 0 && b_cs > 0 && ldc >= N, "batched_gemm: bad strides");
  TCH_CHECK_ARG(causal >= 0 && causal <= 3, "batched_gemm: causal must be 0..3");
  TCH_CHECK_ARG(causal != 1 || M == N, "batched_gemm: causal form 1 needs a square output");
  TCH_CHECK_ARG(causal < 2 || M == K, "batched_gemm: causal forms 2 and 3 need a square A");
  BgemmArgs g{a, b, c, M, N, K, a_rs, a_cs, b_rs, b_cs, ldc, batch_inner, a_bo, a_bi, b_bo, b_bi, c_bo, c_bi, alpha,
              accumulate, causal, (M + kTile - 1) / kTile, (N + kTile - 1) / kTile};
  const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  TCH_CHECK_ARG(tiles <= 0x7fffffff, "batched_gemm: grid out of range");
  const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(batch_outer * batch_inner));
  const double flops = 2.0 * M * N * static_cast<double>(K) * batch_outer * batch_inner * (causal ? 0.5 : 1.0);
  // the profiler's name says which way each operand is contiguous (k: along the reduction, t: across it)
  static const char* const names[2][4] = {
      {"bgemm_kernel<f32,kk>", "bgemm_kernel<f32,kt>", "bgemm_kernel<f32,tk>", "bgemm_kernel<f32,tt>"},
      {"bgemm_kernel<bf16,kk>", "bgemm_kernel<bf16,kt>", "bgemm_kernel<bf16,tk>", "bgemm_kernel<bf16,tt>"}};
  const char* name = names[dtype == kBF16][(a_cs == 1 ? 0 : 2) + (b_cs == 1 ? 0 : 1)];
  return dtype == kBF16 ? launch(ctx, bgemm_kernel<bf16>, grid, dim3(256), g, name, flops, 0)
                        : launch(ctx, bgemm_kernel<float>, grid, dim3(256), g, name, flops, 0);
}

}  // namespace tch
