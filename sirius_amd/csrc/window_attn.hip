// Window attention of the Swin-B step as one launch per direction (bf16, heads 32 wide, at most 64 tokens per
// window): softmax(scale * q k^T + relative position bias [+ shift mask]) v for every (window, head), as written
// out in the reference's train/swin_b_tiny.py:94-110 and run by torchvision's shifted_window_attention for
// train/swin_b.py:38.  A (window, head) problem is 49 x 49 x 32: as separate batched GEMM and softmax launches
// most of each tile is padding and every intermediate makes a round trip through memory.
//
// Two wavefronts share one problem (four per workgroup = two heads of one window).  Its token rows are staged in
// LDS once, padded with zero rows to 64; each wave of the pair owns 32 query rows (forward, first backward
// phase) or 32 key rows (second backward phase) as the lane dimension of its accumulators, so that softmax
// statistics stay per lane (see attn_frag.h for the operand layouts).
//
//   forward    S^T = K Q^T, softmax over the registers, probabilities kept (bf16, rows padded to 64 keys) for
//              the backward, O^T = V^T P^T
//   backward   phase 1 (lane = query): dP^T = V dO^T, delta = sum_k P dP, dS = P (dP - delta), dQ^T = K^T dS^T;
//              dS goes to memory (its sum over windows is the bias gradient) and, with P, to LDS as [query][key]
//              phase 2 (lane = key):   dV^T = dO^T P, dK^T = Q^T dS, both operands read by transposing loads
//
// The bias arrives gathered per head as [heads][64][64] fp32 with -inf in the key columns beyond the window's
// tokens (that is what masks the padding); the shift mask as [windows per image][64][64] fp32.
#include "attn_frag.h"
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

constexpr int kTok = 64;             // padded tokens per window
constexpr int kHd = 32;              // head width
constexpr int kRowS = 80;            // LDS bytes per [token][32] row: 64 + 16 so that 16 rows at one column offset
                                     // fall into different banks
constexpr int kRowP = 144;           // LDS bytes per [query][64 keys] row
constexpr int kTileS = kTok * kRowS; // 5120
constexpr int kTileP = kTok * kRowP; // 9216
constexpr int kPatch = 32 * kRowS;   // 2560: one wave's output rows on their way to memory

struct WinAttnArgs {
  const bf16* qkv;     // [windows * N][3C]
  bf16* o;             // [windows * N][C]                   forward
  bf16* probs;         // [windows * heads][N][64]
  const float* bias;   // [heads][64][64]
  const float* mask;   // [nW][64][64] or null
  const bf16* dout;    // [windows * N][C]                   backward
  bf16* dqkv;          // [windows * N][3C]
  bf16* ds;            // [windows * heads][N][64]
  int heads, N, C, nW;
  float scale;
};

// rows [0, N) of one head's [N][32] slice (row stride `rs` elements) into a zero-padded [64][32] LDS tile, by the
// 128 threads of a wave pair
__device__ inline void stage_rows(const bf16* base, int64_t rs, int N, unsigned char* tile, int t2) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = t2 + 128 * i;
    const int row = c >> 2, slot = c & 3;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (row < N) v = *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(row) * rs + slot * 8);
    *reinterpret_cast<uint4*>(tile + row * kRowS + slot * 16) = v;
  }
}

// acc = result^T: column 8 (r / 4) + 4 (lane / 32) + r % 4 of row lane % 32; rows first .. first+31 of which
// those below N exist, 32 columns, row stride rs
__device__ inline void store_rows(const f32x16_t& acc, float mul, unsigned char* patch, bf16* base, int64_t rs, int first,
                                  int N, int lane) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint2 w;
    w.x = pack_bf16(acc[4 * j] * mul, acc[4 * j + 1] * mul);
    w.y = pack_bf16(acc[4 * j + 2] * mul, acc[4 * j + 3] * mul);
    *reinterpret_cast<uint2*>(patch + (lane & 31) * kRowS + (8 * j + 4 * (lane >> 5)) * 2) = w;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = lane + 64 * i;
    const int row = first + (q >> 2);
    if (row < N)
      *reinterpret_cast<uint4*>(base + static_cast<int64_t>(row) * rs + (q & 3) * 8) =
          *reinterpret_cast<const uint4*>(patch + (q >> 2) * kRowS + (q & 3) * 16);
  }
}

__global__ __launch_bounds__(256) void window_attn_fwd_kernel(WinAttnArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * 2 * kTileS + 4 * kPatch];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int pair = wave >> 1, wp = wave & 1;
  const int pidx = blockIdx.x * 2 + pair;
  const int win = pidx / p.heads, h = pidx - win * p.heads;
  unsigned char* kt = lds + pair * 2 * kTileS;
  unsigned char* vt = kt + kTileS;
  unsigned char* patch = lds + 4 * kTileS + wave * kPatch;
  const int64_t rs = 3 * static_cast<int64_t>(p.C);
  const bf16* qbase = p.qkv + static_cast<int64_t>(win) * p.N * rs + h * kHd;
  stage_rows(qbase + p.C, rs, p.N, kt, tid & 127);
  stage_rows(qbase + 2 * p.C, rs, p.N, vt, tid & 127);

  const int query = 32 * wp + (lane & 31);
  const bool live = query < p.N;
  Chunk qf[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    qf[ks] = zero_chunk();
    if (live) qf[ks].u = *reinterpret_cast<const uint4*>(qbase + static_cast<int64_t>(query) * rs + ks * 16 + 8 * half);
  }
  __syncthreads();

  f32x16_t s[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    zero_acc(s[t]);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) s[t] = mma16(frag_rows<kRowS>(kt, 32 * t, ks, lane), qf[ks], s[t]);
  }
  const float* brow = p.bias + (static_cast<int64_t>(h) * kTok + query) * kTok;
  const float* mrow = p.mask ? p.mask + (static_cast<int64_t>(win % p.nW) * kTok + query) * kTok : nullptr;
  float pr[2][16];
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = 32 * t + 8 * j + 4 * half;
      float4 b = *reinterpret_cast<const float4*>(brow + col);
      if (mrow) {
        const float4 m = *reinterpret_cast<const float4*>(mrow + col);
        b.x += m.x;
        b.y += m.y;
        b.z += m.z;
        b.w += m.w;
      }
      pr[t][4 * j] = s[t][4 * j] * p.scale + b.x;
      pr[t][4 * j + 1] = s[t][4 * j + 1] * p.scale + b.y;
      pr[t][4 * j + 2] = s[t][4 * j + 2] * p.scale + b.z;
      pr[t][4 * j + 3] = s[t][4 * j + 3] * p.scale + b.w;
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, pr[t][4 * j + i]);
    }
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      pr[t][r] = __expf(pr[t][r] - mx);
      sum += pr[t][r];
    }
  sum += __shfl_xor(sum, 32, 64);
  const float inv = 1.f / sum;
  bf16* prow = p.probs + (static_cast<int64_t>(pidx) * p.N + query) * kTok;
  f32x16_t acc;
  zero_acc(acc);
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) pr[t][r] *= inv;
#pragma unroll
    for (int sl = 0; sl < 2; ++sl) {
      const Chunk pc = pack_slab(&pr[t][8 * sl]);
      if (live) {
        *reinterpret_cast<uint2*>(prow + 32 * t + 16 * sl + 4 * half) = make_uint2(pc.w[0], pc.w[1]);
        *reinterpret_cast<uint2*>(prow + 32 * t + 16 * sl + 8 + 4 * half) = make_uint2(pc.w[2], pc.w[3]);
      }
      acc = mma16(frag_cols<kRowS>(vt, 32 * t + 16 * sl, 0, lane), pc, acc);
    }
  }
  store_rows(acc, 1.f, patch, p.o + static_cast<int64_t>(win) * p.N * p.C + h * kHd, p.C, 32 * wp, p.N, lane);
}

__global__ __launch_bounds__(256) void window_attn_bwd_kernel(WinAttnArgs p) {
  constexpr int kPerPair = 4 * kTileS + 2 * kTileP;
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kPerPair];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int pair = wave >> 1, wp = wave & 1;
  const int pidx = blockIdx.x * 2 + pair;
  const int win = pidx / p.heads, h = pidx - win * p.heads;
  unsigned char* qt = lds + pair * kPerPair;
  unsigned char* kt = qt + kTileS;
  unsigned char* vt = kt + kTileS;
  unsigned char* dot = vt + kTileS;
  unsigned char* pt = dot + kTileS;      // P  as [query][key]
  unsigned char* dst = pt + kTileP;      // dS as [query][key]
  unsigned char* patch = kt + wp * kPatch;   // free once both waves of the pair are through phase 1
  const int64_t rs = 3 * static_cast<int64_t>(p.C);
  const int64_t row0 = static_cast<int64_t>(win) * p.N;
  const bf16* qbase = p.qkv + row0 * rs + h * kHd;
  const bf16* dobase = p.dout + row0 * p.C + h * kHd;
  stage_rows(qbase, rs, p.N, qt, tid & 127);
  stage_rows(qbase + p.C, rs, p.N, kt, tid & 127);
  stage_rows(qbase + 2 * p.C, rs, p.N, vt, tid & 127);
  stage_rows(dobase, p.C, p.N, dot, tid & 127);

  // ---- phase 1: this wave's 32 queries ----
  const int query = 32 * wp + (lane & 31);
  const bool live = query < p.N;
  float pr[2][16];
  {
    const bf16* prow = p.probs + (static_cast<int64_t>(pidx) * p.N + query) * kTok;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint2 w = make_uint2(0u, 0u);
        if (live) w = *reinterpret_cast<const uint2*>(prow + 32 * t + 8 * j + 4 * half);
        pr[t][4 * j] = __uint_as_float(w.x << 16);
        pr[t][4 * j + 1] = __uint_as_float(w.x & 0xffff0000u);
        pr[t][4 * j + 2] = __uint_as_float(w.y << 16);
        pr[t][4 * j + 3] = __uint_as_float(w.y & 0xffff0000u);
      }
  }
  __syncthreads();
  f32x16_t dp[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    zero_acc(dp[t]);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      dp[t] = mma16(frag_rows<kRowS>(vt, 32 * t, ks, lane), frag_rows<kRowS>(dot, 32 * wp, ks, lane), dp[t]);
  }
  float delta = 0.f;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) delta += pr[t][r] * dp[t][r];
  delta += __shfl_xor(delta, 32, 64);
  bf16* dsrow = p.ds + (static_cast<int64_t>(pidx) * p.N + query) * kTok;
  f32x16_t dq;
  zero_acc(dq);
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    float ds[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) ds[r] = pr[t][r] * (dp[t][r] - delta);
#pragma unroll
    for (int sl = 0; sl < 2; ++sl) {
      const Chunk pc = pack_slab(&pr[t][8 * sl]);
      const Chunk dc = pack_slab(&ds[8 * sl]);
      const int col = 32 * t + 16 * sl + 4 * half;
      if (live) {
        *reinterpret_cast<uint2*>(dsrow + col) = make_uint2(dc.w[0], dc.w[1]);
        *reinterpret_cast<uint2*>(dsrow + col + 8) = make_uint2(dc.w[2], dc.w[3]);
      }
      *reinterpret_cast<uint2*>(pt + query * kRowP + col * 2) = make_uint2(pc.w[0], pc.w[1]);
      *reinterpret_cast<uint2*>(pt + query * kRowP + (col + 8) * 2) = make_uint2(pc.w[2], pc.w[3]);
      *reinterpret_cast<uint2*>(dst + query * kRowP + col * 2) = make_uint2(dc.w[0], dc.w[1]);
      *reinterpret_cast<uint2*>(dst + query * kRowP + (col + 8) * 2) = make_uint2(dc.w[2], dc.w[3]);
      dq = mma16(frag_cols<kRowS>(kt, 32 * t + 16 * sl, 0, lane), dc, dq);
    }
  }
  __syncthreads();   // P and dS of all 64 queries are in LDS; K and V are no longer read
  store_rows(dq, p.scale, patch, p.dqkv + row0 * rs + h * kHd, rs, 32 * wp, p.N, lane);

  // ---- phase 2: this wave's 32 keys ----
  f32x16_t dk, dv;
  zero_acc(dk);
  zero_acc(dv);
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) {
    dv = mma16(frag_cols<kRowS>(dot, 16 * sl, 0, lane), frag_cols<kRowP>(pt, 16 * sl, wp, lane), dv);
    dk = mma16(frag_cols<kRowS>(qt, 16 * sl, 0, lane), frag_cols<kRowP>(dst, 16 * sl, wp, lane), dk);
  }
  store_rows(dk, p.scale, patch, p.dqkv + row0 * rs + p.C + h * kHd, rs, 32 * wp, p.N, lane);
  store_rows(dv, 1.f, patch, p.dqkv + row0 * rs + 2 * p.C + h * kHd, rs, 32 * wp, p.N, lane);
}

int check_window(const char* who, int dtype, int windows, int heads, int N, int C, int nW) {
  const std::string w(who);
  TCH_CHECK_ARG(dtype == kBF16, w + ": bf16 only");
  TCH_CHECK_ARG(windows >= 1 && heads >= 2 && heads % 2 == 0 && C == heads * kHd, w + ": heads must be 32 wide and even in number");
  TCH_CHECK_ARG(N >= 1 && N <= kTok, w + ": at most 64 tokens per window");
  TCH_CHECK_ARG(nW >= 1 && windows % nW == 0, w + ": the window count must be a multiple of the windows per image");
  TCH_CHECK_ARG(static_cast<int64_t>(windows) * N * 3 * C < (1ll << 31), w + ": tensor too large");
  return 0;
}

}  // namespace

int window_attn_fwd(Context* ctx, int dtype, const void* qkv, void* o, void* probs, const float* bias, const float* mask,
                    int windows, int heads, int N, int C, int nW, float scale) {
  if (int rc = check_window("window_attn_fwd", dtype, windows, heads, N, C, nW)) return rc;
  TCH_CHECK_ARG(qkv && o && probs && bias, "window_attn_fwd: null tensor");
  TCH_CHECK_ARG(((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(o) | reinterpret_cast<uintptr_t>(probs) |
                  reinterpret_cast<uintptr_t>(bias) | reinterpret_cast<uintptr_t>(mask)) & 15) == 0,
                "window_attn_fwd: tensors must be 16-byte aligned");
  WinAttnArgs a{};
  a.qkv = static_cast<const bf16*>(qkv);
  a.o = static_cast<bf16*>(o);
  a.probs = static_cast<bf16*>(probs);
  a.bias = bias;
  a.mask = mask;
  a.heads = heads;
  a.N = N;
  a.C = C;
  a.nW = nW;
  a.scale = scale;
  const double flops = 4.0 * windows * heads * static_cast<double>(N) * N * kHd;
  return launch(ctx, window_attn_fwd_kernel, dim3(windows * heads / 2), dim3(256), a, "window_attn_fwd", flops, 0);
}

int window_attn_bwd(Context* ctx, int dtype, const void* qkv, const void* probs, const void* dout, void* dqkv, void* ds,
                    int windows, int heads, int N, int C, float scale) {
  if (int rc = check_window("window_attn_bwd", dtype, windows, heads, N, C, 1)) return rc;
  TCH_CHECK_ARG(qkv && probs && dout && dqkv && ds, "window_attn_bwd: null tensor");
  TCH_CHECK_ARG(((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(probs) | reinterpret_cast<uintptr_t>(dout) |
                  reinterpret_cast<uintptr_t>(dqkv) | reinterpret_cast<uintptr_t>(ds)) & 15) == 0,
                "window_attn_bwd: tensors must be 16-byte aligned");
  WinAttnArgs a{};
  a.qkv = static_cast<const bf16*>(qkv);
  a.probs = static_cast<bf16*>(const_cast<void*>(probs));
  a.dout = static_cast<const bf16*>(dout);
  a.dqkv = static_cast<bf16*>(dqkv);
  a.ds = static_cast<bf16*>(ds);
  a.heads = heads;
  a.N = N;
  a.C = C;
  a.nW = 1;
  a.scale = scale;
  const double flops = 8.0 * windows * heads * static_cast<double>(N) * N * kHd;
  return launch(ctx, window_attn_bwd_kernel, dim3(windows * heads / 2), dim3(256), a, "window_attn_bwd", flops, 0);
}

}  // namespace tch
