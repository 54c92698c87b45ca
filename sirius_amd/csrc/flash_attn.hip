// Fused attention for the GPT-2 step (bf16, head width 64): softmax(scale * Q K^T [+ causal mask]) V and its
// backward without ever writing the [T, T] score matrix.  What the reference runs here is transformers'
// GPT2Attention inside train/gpt2.py:26 (scores, mask, softmax, dropout p = 0 in the benchmark, context).
//
// Three kernels, all built from the same two MFMA products per step.  In each of them the workgroup keeps one
// side of the problem fixed (128 rows, 32 per wavefront, fragments in registers for the whole kernel) and walks
// over the other side in tiles of 64 rows staged in LDS:
//
//   forward   fixed: 32 queries / wave     walks keys     S^T = K Q^T,  O^T += V^T P^T
//   dQ        fixed: 32 queries / wave     walks keys     S^T, dP^T = V dO^T,  dQ^T += K^T dS^T
//   dK, dV    fixed: 32 keys / wave        walks queries  S = Q K^T, dP = dO V^T,  dV^T += dO^T P,  dK^T += Q^T dS
//
// The products are oriented so that the fixed side is the lane dimension of the 32x32 accumulator (lane % 32 =
// the fixed row, registers = the walked rows).  A row statistic of the fixed side (running maximum, sum, the
// saved log-sum-exp, delta = sum_d dO*O) is then one scalar per lane, a reduction over the walked rows runs over
// the lane's own registers plus one exchange with lane ^ 32, and the probabilities are already laid out as the
// second operand of the next product: the accumulator's registers 8s .. 8s+7 of a lane are 8 walked rows
// {16s + 8t + 4(lane/32) + i}, which is a permutation of the 16 reduction indices of one MFMA step; the other
// operand is read from LDS with the same permutation (transposing reads, ds_read_b64_tr_b16).
//
// Numerics: scores and statistics in fp32 from the bf16 products, exponentials as exp2 of pre-scaled values,
// probabilities rounded to bf16 for the second product (as the unfused path stores them).  The backward
// recomputes the probabilities from the saved log-sum-exp; dQ and (dK, dV) are two launches so that nothing is
// accumulated atomically and results do not depend on scheduling.
#include "attn_frag.h"
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

constexpr int kHd = 64;          // head width
constexpr int kFixed = 128;      // rows of the fixed side per workgroup
constexpr int kWalk = 64;        // rows of the walked side per step
constexpr int kRowB = 144;       // LDS bytes per tile row: 64 bf16 + 16 bytes, so that 16 rows at one column
                                 // offset and the 4 x 32-byte patches of a transposing read spread over the banks
constexpr int kTileB = kWalk * kRowB;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct FlashArgs {
  const bf16* q;
  const bf16* k;
  const bf16* v;
  const bf16* o;      // backward
  const bf16* dout;   // backward
  bf16* out;          // forward: o; dQ kernel: dq
  bf16* dk;
  bf16* dv;
  float* lse;         // [B * H][T], natural logarithm
  float* delta;       // [B * H][T]
  int64_t qkv_rs, qkv_bs;   // row / sample strides of q, k, v, dq, dk, dv (elements); head h starts at column 64 h
  int64_t o_rs, o_bs;       // the same for o and dout
  int H, T;
  float scale;
};

// a [64][64] bf16 tile: global -> registers (two 16-byte chunks per thread) -> LDS rows of kRowB bytes
struct TileRegs {
  uint4 lo, hi;   // rows tid / 8 and 32 + tid / 8, slot tid % 8 (plain members: an array here ends up in scratch)
};
__device__ inline TileRegs tile_load(const bf16* base, int64_t rs, int tid) {
  const bf16* src = base + static_cast<int64_t>(tid >> 3) * rs + (tid & 7) * 8;
  TileRegs r;
  r.lo = *reinterpret_cast<const uint4*>(src);
  r.hi = *reinterpret_cast<const uint4*>(src + 32 * rs);
  return r;
}
__device__ inline void tile_store(unsigned char* lds, int tid, const TileRegs& r) {
  unsigned char* dst = lds + (tid >> 3) * kRowB + (tid & 7) * 16;
  *reinterpret_cast<uint4*>(dst) = r.lo;
  *reinterpret_cast<uint4*>(dst + 32 * kRowB) = r.hi;
}

// this wave's fragments of 32 fixed rows (row = first + lane % 32): 4 chunks cover the lane half's 32 columns
__device__ inline void load_fixed(const bf16* base, int64_t rs, int first, int lane, Chunk (&f)[4]) {
  const bf16* row = base + static_cast<int64_t>(first + (lane & 31)) * rs + 8 * (lane >> 5);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) f[ks].u = *reinterpret_cast<const uint4*>(row + ks * 16);
}

// acc[ct] holds the transposed result: column 32 ct + 8 (r / 4) + 4 (lane / 32) + r % 4 of fixed row lane % 32.
// Goes through this wave's LDS patch so that a row leaves as 16-byte pieces.
__device__ inline void store_fixed(f32x16_t (&acc)[2], float mul, unsigned char* patch, bf16* base, int64_t rs, int first,
                                   int lane) {
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint2 w;
      w.x = pack_bf16(acc[ct][4 * j] * mul, acc[ct][4 * j + 1] * mul);
      w.y = pack_bf16(acc[ct][4 * j + 2] * mul, acc[ct][4 * j + 3] * mul);
      *reinterpret_cast<uint2*>(patch + (lane & 31) * kRowB + (32 * ct + 8 * j + 4 * (lane >> 5)) * 2) = w;
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = lane + 64 * i;
    const uint4 v = *reinterpret_cast<const uint4*>(patch + (q >> 3) * kRowB + (q & 7) * 16);
    *reinterpret_cast<uint4*>(base + static_cast<int64_t>(first + (q >> 3)) * rs + (q & 7) * 8) = v;
  }
}

// ---------------------------------------------------------------------------------------------------------
// forward (DQ = false) and the dQ half of the backward (DQ = true): fixed queries, walked keys
// ---------------------------------------------------------------------------------------------------------
template <bool CAUSAL, bool DQ>
__global__ __launch_bounds__(256) void flash_query_kernel(FlashArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kTileB];
  unsigned char* kt = lds;
  unsigned char* vt = lds + kTileB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  // Workgroup ids go to the XCDs round-robin and all of them are resident at once, so the order is the
  // placement: the blocks of one head keep one residue of the id modulo 8 (one XCD, one L2 for its keys and
  // values), and the long blocks of a causal problem come first so that each compute unit's share of
  // consecutive ids mixes long and short ones.
  const int nbh = gridDim.x / (p.T / kFixed);
  const int qb = p.T / kFixed - 1 - blockIdx.x / nbh;
  const int bh = blockIdx.x % nbh;
  const int b = bh / p.H, h = bh - b * p.H;
  const int64_t qkv_off = b * p.qkv_bs + h * kHd, o_off = b * p.o_bs + h * kHd;
  const int q0 = qb * kFixed, qw0 = q0 + 32 * wave;
  const int query = qw0 + (lane & 31);

  Chunk qf[4], dof[4];
  load_fixed(p.q + qkv_off, p.qkv_rs, qw0, lane, qf);
  float lse2 = 0.f, delta = 0.f;
  if (DQ) {
    load_fixed(p.dout + o_off, p.o_rs, qw0, lane, dof);
    Chunk of[4];
    load_fixed(p.o + o_off, p.o_rs, qw0, lane, of);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      float a[8], g[8];
      chunk_to_float<bf16>(of[ks], a);
      chunk_to_float<bf16>(dof[ks], g);
#pragma unroll
      for (int e = 0; e < 8; ++e) delta += a[e] * g[e];
    }
    delta += __shfl_xor(delta, 32, 64);
    if (half == 0) p.delta[static_cast<int64_t>(bh) * p.T + query] = delta;
    lse2 = p.lse[static_cast<int64_t>(bh) * p.T + query] * kLog2e;
  }

  const int steps = CAUSAL ? (q0 + kFixed) / kWalk : p.T / kWalk;
  const bf16* kbase = p.k + qkv_off;
  const bf16* vbase = p.v + qkv_off;
  TileRegs rk = tile_load(kbase, p.qkv_rs, tid);
  TileRegs rv = tile_load(vbase, p.qkv_rs, tid);

  f32x16_t acc[2];
  zero_acc(acc[0]);
  zero_acc(acc[1]);
  const float c = p.scale * kLog2e;
  float m = -INFINITY, l = 0.f;

  for (int kb = 0; kb < steps; ++kb) {
    __syncthreads();
    tile_store(kt, tid, rk);
    tile_store(vt, tid, rv);
    __syncthreads();
    {
      // the last step fetches its own tile again rather than branching around the loads
      const int64_t next = static_cast<int64_t>(kb + 1 < steps ? kb + 1 : kb) * kWalk * p.qkv_rs;
      rk = tile_load(kbase + next, p.qkv_rs, tid);
      rv = tile_load(vbase + next, p.qkv_rs, tid);
    }
    const int k0 = kb * kWalk;
    if (CAUSAL && k0 > qw0 + 31) continue;   // nothing of this tile is visible to this wave's queries

    f32x16_t s[2], dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      zero_acc(s[t]);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) s[t] = mma16(frag_rows<kRowB>(kt, 32 * t, ks, lane), qf[ks], s[t]);
      if (DQ) {
        zero_acc(dp[t]);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) dp[t] = mma16(frag_rows<kRowB>(vt, 32 * t, ks, lane), dof[ks], dp[t]);
      }
    }
    const bool diagonal = CAUSAL && k0 + kWalk - 1 > qw0;   // some key of the tile lies beyond some query
    float pr[2][16];
    if (!DQ) {
      // running maximum on the raw scores (the scale is positive), then exp2(s * c - m * c) as one fused
      // multiply-add and one exponential per score
      float bmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = s[t][r];
          if (diagonal && k0 + 32 * t + 8 * (r >> 2) + 4 * half + (r & 3) > query) v = -INFINITY;
          pr[t][r] = v;
          bmax = fmaxf(bmax, v);
        }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
      const float m_new = fmaxf(m, bmax);
      const bool moved = m_new != m;
      const float alpha = __builtin_amdgcn_exp2f((m - m_new) * c);
      m = m_new;
      const float mc = m_new * c;
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          pr[t][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(pr[t][r], c, -mc));
          sum += pr[t][r];
        }
      l = l * alpha + sum;
      // after the first tiles the maxima seldom move: the accumulators are rescaled only when one in the wave did
      if (__any(moved)) {
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[ct][e] *= alpha;
      }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float pv = __builtin_amdgcn_exp2f(s[t][r] * c - lse2);
          if (diagonal && k0 + 32 * t + 8 * (r >> 2) + 4 * half + (r & 3) > query) pv = 0.f;
          pr[t][r] = pv * (dp[t][r] - delta);
        }
    }
    const unsigned char* second = DQ ? kt : vt;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const Chunk pc = pack_slab(&pr[t][8 * sl]);
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[ct] = mma16(frag_cols<kRowB>(second, 32 * t + 16 * sl, ct, lane), pc, acc[ct]);
      }
  }

  float mul = p.scale;
  if (!DQ) {
    l += __shfl_xor(l, 32, 64);
    mul = 1.f / l;
    if (half == 0) p.lse[static_cast<int64_t>(bh) * p.T + query] = m * p.scale + __builtin_amdgcn_logf(l) * kLn2;
  }
  __syncthreads();   // every wave is done with the tiles: the space becomes four output patches
  store_fixed(acc, mul, lds + wave * 32 * kRowB, p.out + (DQ ? qkv_off : o_off), DQ ? p.qkv_rs : p.o_rs, qw0, lane);
}

// ---------------------------------------------------------------------------------------------------------
// dK and dV: fixed keys, walked queries
// ---------------------------------------------------------------------------------------------------------
template <bool CAUSAL>
__global__ __launch_bounds__(256) void flash_key_kernel(FlashArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kTileB];
  __shared__ __attribute__((aligned(16))) float stat[2][kWalk];   // log-sum-exp (base 2) and delta of the staged queries
  unsigned char* qt = lds;
  unsigned char* dot = lds + kTileB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int nbh = gridDim.x / (p.T / kFixed);   // placement as in flash_query_kernel: early keys see most queries
  const int kblk = blockIdx.x / nbh;
  const int bh = blockIdx.x % nbh;
  const int b = bh / p.H, h = bh - b * p.H;
  const int64_t qkv_off = b * p.qkv_bs + h * kHd, o_off = b * p.o_bs + h * kHd;
  const int k0 = kblk * kFixed, kw0 = k0 + 32 * wave;
  const int key = kw0 + (lane & 31);

  Chunk kf[4], vf[4];
  load_fixed(p.k + qkv_off, p.qkv_rs, kw0, lane, kf);
  load_fixed(p.v + qkv_off, p.qkv_rs, kw0, lane, vf);

  const int first = CAUSAL ? k0 / kWalk : 0;   // queries before the first key see none of these keys
  const int steps = p.T / kWalk;
  const bf16* qbase = p.q + qkv_off;
  const bf16* dobase = p.dout + o_off;
  const float* lse = p.lse + static_cast<int64_t>(bh) * p.T;
  const float* dlt = p.delta + static_cast<int64_t>(bh) * p.T;
  TileRegs rq, rd;
  float rstat = 0.f;
  auto fetch = [&](int qb) {
    rq = tile_load(qbase + static_cast<int64_t>(qb) * kWalk * p.qkv_rs, p.qkv_rs, tid);
    rd = tile_load(dobase + static_cast<int64_t>(qb) * kWalk * p.o_rs, p.o_rs, tid);
    if (tid < kWalk) rstat = lse[qb * kWalk + tid] * kLog2e;
    else if (tid < 2 * kWalk) rstat = dlt[qb * kWalk + tid - kWalk];
  };
  fetch(first);

  f32x16_t dk[2], dv[2];
  zero_acc(dk[0]);
  zero_acc(dk[1]);
  zero_acc(dv[0]);
  zero_acc(dv[1]);
  const float c = p.scale * kLog2e;

  for (int qb = first; qb < steps; ++qb) {
    __syncthreads();
    tile_store(qt, tid, rq);
    tile_store(dot, tid, rd);
    if (tid < 2 * kWalk) stat[tid >> 6][tid & 63] = rstat;
    __syncthreads();
    fetch(qb + 1 < steps ? qb + 1 : qb);   // the last step fetches its own tile again: no branch around the loads
    const int q0 = qb * kWalk;
    if (CAUSAL && q0 + kWalk - 1 < kw0) continue;   // every staged query lies before this wave's keys

    f32x16_t s[2], dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      zero_acc(s[t]);
      zero_acc(dp[t]);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        s[t] = mma16(frag_rows<kRowB>(qt, 32 * t, ks, lane), kf[ks], s[t]);
        dp[t] = mma16(frag_rows<kRowB>(dot, 32 * t, ks, lane), vf[ks], dp[t]);
      }
    }
    const bool diagonal = CAUSAL && q0 < kw0 + 31;   // some staged query lies before some key of this wave
    float pr[2][16], ds[2][16];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int row = 32 * t + 8 * j + 4 * half;
        const float4 l4 = *reinterpret_cast<const float4*>(&stat[0][row]);
        const float4 d4 = *reinterpret_cast<const float4*>(&stat[1][row]);
        const float ls[4] = {l4.x, l4.y, l4.z, l4.w}, dl[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 4 * j + i;
          float pv = __builtin_amdgcn_exp2f(s[t][r] * c - ls[i]);
          if (diagonal && key > q0 + row + i) pv = 0.f;
          pr[t][r] = pv;
          ds[t][r] = pv * (dp[t][r] - dl[i]);
        }
      }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const Chunk pc = pack_slab(&pr[t][8 * sl]);
        const Chunk dc = pack_slab(&ds[t][8 * sl]);
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
          dv[ct] = mma16(frag_cols<kRowB>(dot, 32 * t + 16 * sl, ct, lane), pc, dv[ct]);
          dk[ct] = mma16(frag_cols<kRowB>(qt, 32 * t + 16 * sl, ct, lane), dc, dk[ct]);
        }
      }
  }
  __syncthreads();
  unsigned char* patch = lds + wave * 32 * kRowB;
  store_fixed(dv, 1.f, patch, p.dv + qkv_off, p.qkv_rs, kw0, lane);
  __syncthreads();
  store_fixed(dk, p.scale, patch, p.dk + qkv_off, p.qkv_rs, kw0, lane);
}

int check_geometry(const char* who, int dtype, int B, int H, int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs,
                   int64_t o_bs) {
  const std::string w(who);
  TCH_CHECK_ARG(dtype == kBF16, w + ": bf16 only");
  TCH_CHECK_ARG(B >= 1 && H >= 1 && T >= kFixed && T % kFixed == 0, w + ": the sequence length must be a multiple of 128");
  TCH_CHECK_ARG(static_cast<int64_t>(B) * H * (T / kFixed) < (1ll << 31), w + ": too many blocks for one grid");
  TCH_CHECK_ARG(qkv_rs >= static_cast<int64_t>(H) * kHd && o_rs >= static_cast<int64_t>(H) * kHd,
                w + ": row strides shorter than the heads");
  TCH_CHECK_ARG(qkv_rs % 8 == 0 && qkv_bs % 8 == 0 && o_rs % 8 == 0 && o_bs % 8 == 0,
                w + ": strides must keep 16-byte alignment");
  return 0;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

}  // namespace

int flash_attn_fwd(Context* ctx, int dtype, const void* q, const void* k, const void* v, void* o, float* lse, int B,
                   int H, int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal) {
  if (int rc = check_geometry("flash_attn_fwd", dtype, B, H, T, qkv_rs, qkv_bs, o_rs, o_bs)) return rc;
  TCH_CHECK_ARG(q && k && v && o && lse, "flash_attn_fwd: null tensor");
  TCH_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o), "flash_attn_fwd: tensors must be 16-byte aligned");
  FlashArgs a{};
  a.q = static_cast<const bf16*>(q);
  a.k = static_cast<const bf16*>(k);
  a.v = static_cast<const bf16*>(v);
  a.out = static_cast<bf16*>(o);
  a.lse = lse;
  a.qkv_rs = qkv_rs;
  a.qkv_bs = qkv_bs;
  a.o_rs = o_rs;
  a.o_bs = o_bs;
  a.H = H;
  a.T = T;
  a.scale = scale;
  const dim3 grid(static_cast<unsigned>(T / kFixed) * B * H);
  const double flops = 4.0 * B * H * static_cast<double>(T) * T * kHd * (causal ? 0.5 : 1.0);
  return causal ? launch(ctx, flash_query_kernel<true, false>, grid, dim3(256), a, "flash_attn_fwd<causal>", flops, 0)
                : launch(ctx, flash_query_kernel<false, false>, grid, dim3(256), a, "flash_attn_fwd<full>", flops, 0);
}

int flash_attn_bwd(Context* ctx, int dtype, const void* q, const void* k, const void* v, const void* o, const void* dout,
                   const float* lse, float* delta, void* dq, void* dk, void* dv, int B, int H, int T, int64_t qkv_rs,
                   int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal) {
  if (int rc = check_geometry("flash_attn_bwd", dtype, B, H, T, qkv_rs, qkv_bs, o_rs, o_bs)) return rc;
  TCH_CHECK_ARG(q && k && v && o && dout && lse && delta && dq && dk && dv, "flash_attn_bwd: null tensor");
  TCH_CHECK_ARG(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) && aligned16(dout) && aligned16(dq) &&
                    aligned16(dk) && aligned16(dv),
                "flash_attn_bwd: tensors must be 16-byte aligned");
  FlashArgs a{};
  a.q = static_cast<const bf16*>(q);
  a.k = static_cast<const bf16*>(k);
  a.v = static_cast<const bf16*>(v);
  a.o = static_cast<const bf16*>(o);
  a.dout = static_cast<const bf16*>(dout);
  a.out = static_cast<bf16*>(dq);
  a.dk = static_cast<bf16*>(dk);
  a.dv = static_cast<bf16*>(dv);
  a.lse = const_cast<float*>(lse);
  a.delta = delta;
  a.qkv_rs = qkv_rs;
  a.qkv_bs = qkv_bs;
  a.o_rs = o_rs;
  a.o_bs = o_bs;
  a.H = H;
  a.T = T;
  a.scale = scale;
  const dim3 grid(static_cast<unsigned>(T / kFixed) * B * H);
  const double pair = 2.0 * B * H * static_cast<double>(T) * T * kHd * (causal ? 0.5 : 1.0);   // one T x T x 64 product
  // the dQ launch leaves delta for the dK / dV launch
  int rc = causal ? launch(ctx, flash_query_kernel<true, true>, grid, dim3(256), a, "flash_attn_dq<causal>", 3.0 * pair, 0)
                  : launch(ctx, flash_query_kernel<false, true>, grid, dim3(256), a, "flash_attn_dq<full>", 3.0 * pair, 0);
  if (rc) return rc;
  return causal ? launch(ctx, flash_key_kernel<true>, grid, dim3(256), a, "flash_attn_dkv<causal>", 4.0 * pair, 0)
                : launch(ctx, flash_key_kernel<false>, grid, dim3(256), a, "flash_attn_dkv<full>", 4.0 * pair, 0);
}

}  // namespace tch
