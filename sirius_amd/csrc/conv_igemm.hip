// Implicit-GEMM convolution for gfx950: forward, data gradient and weight
// gradient over NHWC activations and KRSC filters, on the 32x32 MFMA tiles
// (v_mfma_f32_32x32x16_bf16 for bf16 storage, v_mfma_f32_32x32x2_f32 for fp32),
// fp32 accumulation, operands staged through LDS in 16-byte chunks.
//
// The reference has no convolution code of its own: its training scripts call
// torchvision's ResNet (train/resnet152.py:22) and the arithmetic is
// F.conv2d / its autograd formulas.  These kernels restate that arithmetic:
//   FWD    y[n,ho,wo,k]  = sum_{r,s,c} x[n, ho*st-p+r, wo*st-p+s, c] * w[k,r,s,c]
//   DGRAD  dx[n,h,w,c]   = sum_{r,s,k} dy[n,(h+p-r)/st,(w+p-s)/st,k] * w[k,r,s,c]
//   WGRAD  dw[k,r,s,c]   = sum_{n,ho,wo} dy[n,ho,wo,k] * x[n, ho*st-p+r, wo*st-p+s, c]
//
// GEMM view (rows x cols, reduction):
//   FWD    (N*Ho*Wo) x K,        over R*S*C
//   DGRAD  (N*H*W)   x C,        over R*S*K
//   WGRAD  K         x (R*S*C),  over N*Ho*Wo, split across workgroups
//
// A tile row in LDS holds one GEMM row (or column) and BK reduction elements
// = 4 chunks of 16 bytes (+1 chunk of padding).  A lane's MFMA operand is one
// chunk: lanes 0-31 take chunk 2j, lanes 32-63 chunk 2j+1 of their row, so the
// two operands always agree on which reduction elements a lane group holds.
#include "kernels.h"
#include "ops.h"

#include <string>

namespace tch {
namespace {

constexpr int kLdsStride = 5;  // chunks per LDS tile row: 4 data + 1 pad

enum Mode : int { kFwd = 0, kDgrad = 1, kWgrad = 2 };

struct IgemmArgs {
  const void* a_src;  // FWD: x        DGRAD: dy       WGRAD: dy
  const void* b_src;  // FWD: w        DGRAD: w        WGRAD: x
  void* out;          // FWD: y        DGRAD: dx       WGRAD: dw (fp32) or split partials
  const void* add;    // optional addend, laid out like out (FWD/DGRAD)
  const void* mask;   // optional: addend counts only where mask > 0
  const float* bias;  // optional per-column bias (FWD)
  int N, H, W, C;     // x side
  int Ho, Wo, K;      // y side
  int R, S, stride, stride_log2, pad;
  int gemm_m, gemm_n, gemm_k;
  int tiles_m, tiles_n, splits;
  int k_per_split;  // multiple of BK
  int out_f32;      // FWD/DGRAD: store fp32 instead of T
  int accumulate;   // WGRAD with splits == 1: out += result
  int pointwise;    // 1x1, stride 1, pad 0
  FastDiv div_plane;  // pixels per image on the gather side
  FastDiv div_width;  // row width on the gather side
};

template <typename T>
__device__ inline void mma(const Chunk& a, const Chunk& b, f32x16_t& acc);
template <>
__device__ inline void mma<bf16>(const Chunk& a, const Chunk& b, f32x16_t& acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, b.h, acc, 0, 0, 0);
}
template <>
__device__ inline void mma<float>(const Chunk& a, const Chunk& b, f32x16_t& acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[e], b.f[e], acc, 0, 0, 0);
}

__device__ inline Chunk load_chunk(const void* base, int64_t elem_off, int elem_bytes, bool valid) {
  Chunk c = zero_chunk();
  if (valid) c.u = *reinterpret_cast<const uint4*>(static_cast<const char*>(base) + elem_off * elem_bytes);
  return c;
}

// v[j] holds E consecutive elements of memory row j; produce out[e] = the e-th
// element of every row, i.e. the ExE transpose.
template <typename T>
__device__ inline void transpose_block(const Chunk* v, Chunk* out);
template <>
__device__ inline void transpose_block<float>(const Chunk* v, Chunk* out) {
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int q = 0; q < 4; ++q) out[e].w[q] = v[q].w[e];
}
template <>
__device__ inline void transpose_block<bf16>(const Chunk* v, Chunk* out) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int src = e >> 1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t lo = v[2 * q].w[src], hi = v[2 * q + 1].w[src];
      out[e].w[q] = (e & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
    }
  }
}

// Walks the reduction index of a filter-tap-major operand: (tap, channel) with
// `channels` per tap, advancing by BK per step.
struct TapWalker {
  int tap, ch;
  __device__ inline void init(int k, int channels) {
    tap = k / channels;
    ch = k - tap * channels;
  }
  __device__ inline void advance(int step, int channels) {
    ch += step;
    while (ch >= channels) {
      ch -= channels;
      ++tap;
    }
  }
};

template <typename T, int MODE, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM* WN * 64) void igemm_kernel(IgemmArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  constexpr int BK = 4 * E;
  constexpr int BM = WM * TM * 32;
  constexpr int BN = WN * TN * 32;
  constexpr int NT = WM * WN * 64;
  constexpr int EB = sizeof(T);
  // direct loaders: one chunk per (row, chunk-in-row)
  constexpr int A_PT = (BM * 4 + NT - 1) / NT;
  constexpr int B_PT = (BN * 4 + NT - 1) / NT;
  static_assert((BM * 4) % NT == 0 || BM * 4 < NT, "tile/loader mismatch");
  static_assert((BN * 4) % NT == 0 || BN * 4 < NT, "tile/loader mismatch");
  // transposing loaders: one ExE block per active thread
  constexpr int A_BLOCKS = (BM / E) * 4;
  constexpr int B_BLOCKS = (BN / E) * 4;
  static_assert(A_BLOCKS <= NT && B_BLOCKS <= NT, "transposing loader needs one block per thread");

  __shared__ uint4 lds_a[2][BM * kLdsStride];
  __shared__ uint4 lds_b[2][BN * kLdsStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  const uint32_t nwg = gridDim.x;
  uint32_t id = xcd_remap(blockIdx.x, nwg);
  const int tiles_mn = p.tiles_m * p.tiles_n;
  const int split = id / tiles_mn;
  id -= split * tiles_mn;
  const int tile_m = id / p.tiles_n;
  const int tile_n = id - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int k_begin = split * p.k_per_split;
  int k_end = k_begin + p.k_per_split;
  if (k_end > p.gemm_k) k_end = p.gemm_k;
  const int nk = (k_end - k_begin + BK - 1) / BK;

  const int RS = p.R * p.S;

  // ---------------- per-thread loader state ----------------
  // FWD / DGRAD operand A: gather of activation rows
  int a_base[A_PT], a_h0[A_PT], a_w0[A_PT];
  bool a_row_ok[A_PT];
  TapWalker a_walk;  // same chunk column for every i, so one walker
  int in_h = 0, in_w = 0, in_c = 0;
  // FWD operand B: dense filter rows
  // DGRAD operand B / WGRAD operands: transposing loaders
  int t_row0_a = 0, t_kc_a = 0;
  int t_row0_b = 0, t_kc_b = 0;
  bool t_act_a = false, t_act_b = false;
  TapWalker b_walk;
  int wb_r = 0, wb_s = 0, wb_c = 0;  // WGRAD B: this thread's filter tap / channel

  if constexpr (MODE == kFwd || MODE == kDgrad) {
    in_h = (MODE == kFwd) ? p.H : p.Ho;
    in_w = (MODE == kFwd) ? p.W : p.Wo;
    in_c = (MODE == kFwd) ? p.C : p.K;
    const int chunk_col = tid & 3;
    a_walk.init(k_begin + chunk_col * E, in_c);
#pragma unroll
    for (int i = 0; i < A_PT; ++i) {
      int q = tid + i * NT;
      int row = m0 + (q >> 2);
      a_row_ok[i] = (q < BM * 4) && row < p.gemm_m;
      uint32_t img = 0, pix = 0, oh = 0, ow = 0;
      if (a_row_ok[i]) {
        p.div_plane.divmod(static_cast<uint32_t>(row), img, pix);
        p.div_width.divmod(pix, oh, ow);
      }
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
  if constexpr (MODE == kWgrad) {
    t_act_a = tid < A_BLOCKS;
    t_kc_a = tid & 3;
    t_row0_a = m0 + (tid >> 2) * E;
    t_act_b = tid < B_BLOCKS;
    t_kc_b = tid & 3;
    t_row0_b = n0 + (tid >> 2) * E;
    if (t_act_b && t_row0_b < p.gemm_n) {
      int tap = t_row0_b / p.C;
      wb_c = t_row0_b - tap * p.C;
      wb_r = tap / p.S;
      wb_s = tap - wb_r * p.S;
    }
  }

  Chunk ra[(MODE == kWgrad) ? E : A_PT];
  Chunk rb[(MODE == kWgrad) ? E : B_PT];

  auto load_tiles = [&](int kt) {
    const int k0 = k_begin + kt * BK;
    // ---- operand A ----
    if constexpr (MODE == kFwd || MODE == kDgrad) {
      const int r = a_walk.tap / p.S, s = a_walk.tap - r * p.S;
      const bool tap_ok = a_walk.tap < RS && (k0 + (tid & 3) * E) < k_end;
#pragma unroll
      for (int i = 0; i < A_PT; ++i) {
        int hi, wi;
        bool ok = a_row_ok[i] && tap_ok;
        if (MODE == kFwd) {
          hi = a_h0[i] + r;
          wi = a_w0[i] + s;
        } else {
          int th = a_h0[i] - r, tw = a_w0[i] - s;
          int sm = p.stride - 1;
          ok = ok && th >= 0 && tw >= 0 && ((th & sm) == 0) && ((tw & sm) == 0);
          hi = th >> p.stride_log2;
          wi = tw >> p.stride_log2;
        }
        ok = ok && static_cast<unsigned>(hi) < static_cast<unsigned>(in_h) &&
             static_cast<unsigned>(wi) < static_cast<unsigned>(in_w);
        int64_t off = static_cast<int64_t>(a_base[i]) + (hi * in_w + wi) * in_c + a_walk.ch;
        ra[i] = load_chunk(p.a_src, off, EB, ok);
      }
      a_walk.advance(BK, in_c);
    } else {
      // WGRAD A: rows = output channels (contiguous in dy), reduction = pixels
      const int pix0 = k0 + t_kc_a * E;
      const bool ok_rows = t_act_a && t_row0_a < p.gemm_m;
#pragma unroll
      for (int j = 0; j < E; ++j) {
        int pix = pix0 + j;
        bool ok = ok_rows && pix < k_end;
        ra[j] = load_chunk(p.a_src, static_cast<int64_t>(pix) * p.K + t_row0_a, EB, ok);
      }
    }
    // ---- operand B ----
    if constexpr (MODE == kFwd || MODE == kDgrad) {
      // dense filter rows: FWD reads w[K][R*S*C], DGRAD reads the transposed filter wt[C][R*S*K]
#pragma unroll
      for (int i = 0; i < B_PT; ++i) {
        int q = tid + i * NT;
        int row = n0 + (q >> 2);
        int k = k0 + (q & 3) * E;
        bool ok = (q < BN * 4) && row < p.gemm_n && k < k_end;
        rb[i] = load_chunk(p.b_src, static_cast<int64_t>(row) * p.gemm_k + k, EB, ok);
      }
    } else {
      // WGRAD B: rows = (tap, in channel) fixed per thread, reduction = pixels
      const int pix0 = k0 + t_kc_b * E;
      const bool ok_rows = t_act_b && t_row0_b < p.gemm_n;
      if (p.pointwise) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
          int pix = pix0 + j;
          bool ok = ok_rows && pix < k_end;
          rb[j] = load_chunk(p.b_src, static_cast<int64_t>(pix) * p.C + wb_c, EB, ok);
        }
      } else {
        uint32_t img = 0, rem = 0, oh = 0, ow = 0;
        if (pix0 < k_end) {
          p.div_plane.divmod(static_cast<uint32_t>(pix0), img, rem);
          p.div_width.divmod(rem, oh, ow);
        }
        int n = img, ho = oh, wo = ow;
#pragma unroll
        for (int j = 0; j < E; ++j) {
          int hi = ho * p.stride - p.pad + wb_r;
          int wi = wo * p.stride - p.pad + wb_s;
          bool ok = ok_rows && (pix0 + j) < k_end && static_cast<unsigned>(hi) < static_cast<unsigned>(p.H) &&
                    static_cast<unsigned>(wi) < static_cast<unsigned>(p.W);
          int64_t off = (static_cast<int64_t>(n) * p.H * p.W + hi * p.W + wi) * p.C + wb_c;
          rb[j] = load_chunk(p.b_src, off, EB, ok);
          if (++wo == p.Wo) {
            wo = 0;
            if (++ho == p.Ho) {
              ho = 0;
              ++n;
            }
          }
        }
      }
    }
  };

  auto store_tiles = [&](int buf) {
    if constexpr (MODE == kFwd || MODE == kDgrad) {
#pragma unroll
      for (int i = 0; i < A_PT; ++i) {
        int q = tid + i * NT;
        if (q < BM * 4) lds_a[buf][(q >> 2) * kLdsStride + (q & 3)] = ra[i].u;
      }
    } else {
      if (t_act_a) {
        Chunk t[E];
        transpose_block<T>(ra, t);
        int row = (tid >> 2) * E;
#pragma unroll
        for (int e = 0; e < E; ++e) lds_a[buf][(row + e) * kLdsStride + t_kc_a] = t[e].u;
      }
    }
    if constexpr (MODE == kFwd || MODE == kDgrad) {
#pragma unroll
      for (int i = 0; i < B_PT; ++i) {
        int q = tid + i * NT;
        if (q < BN * 4) lds_b[buf][(q >> 2) * kLdsStride + (q & 3)] = rb[i].u;
      }
    } else {
      if (t_act_b) {
        Chunk t[E];
        transpose_block<T>(rb, t);
        int row = (tid >> 2) * E;
#pragma unroll
        for (int e = 0; e < E; ++e) lds_b[buf][(row + e) * kLdsStride + t_kc_b] = t[e].u;
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

  if (nk > 0) {
    load_tiles(0);
    store_tiles(0);
  }
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    const bool more = (kt + 1) < nk;
    if (more) load_tiles(kt + 1);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Chunk fa[TM], fb[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        fa[tm].u = lds_a[buf][((wm * TM + tm) * 32 + frag_row) * kLdsStride + 2 * j + frag_half];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        fb[tn].u = lds_b[buf][((wn * TN + tn) * 32 + frag_row) * kLdsStride + 2 * j + frag_half];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) mma<T>(fa[tm], fb[tn], acc[tm][tn]);
    }
    if (more) store_tiles(buf ^ 1);
    __syncthreads();
  }

  // ---------------- epilogue ----------------
  // 32x32 accumulator: lane owns column (lane % 32); element i sits in row
  // 8*(i/4) + 4*(lane/32) + i%4.
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int col = n0 + (wn * TN + tn) * 32 + frag_row;
      if (col >= p.gemm_n) continue;
      float bias = 0.f;
      if (MODE == kFwd && p.bias) bias = p.bias[col];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = m0 + (wm * TM + tm) * 32 + 8 * (i >> 2) + 4 * frag_half + (i & 3);
        if (row >= p.gemm_m) continue;
        const int64_t idx = static_cast<int64_t>(row) * p.gemm_n + col;
        float v = acc[tm][tn][i];
        if constexpr (MODE == kWgrad) {
          float* o = static_cast<float*>(p.out);
          if (p.splits > 1) {
            o[static_cast<int64_t>(split) * p.gemm_m * p.gemm_n + idx] = v;
          } else {
            o[idx] = p.accumulate ? o[idx] + v : v;
          }
        } else {
          v += bias;
          if (p.add) {
            float a = Elem<T>::load(static_cast<const T*>(p.add) + idx);
            if (p.mask && !(Elem<T>::load(static_cast<const T*>(p.mask) + idx) > 0.f)) a = 0.f;
            v += a;
          }
          if (p.out_f32)
            static_cast<float*>(p.out)[idx] = v;
          else
            Elem<T>::store(static_cast<T*>(p.out) + idx, v);
        }
      }
    }
  }
}

struct ReduceArgs {
  const float* partial;
  float* out;
  int64_t n;
  int splits;
  int accumulate;
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(ReduceArgs p) {
  int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= p.n) return;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < p.splits; ++k) {
    float4 v = *reinterpret_cast<const float4*>(p.partial + static_cast<int64_t>(k) * p.n + i);
    s.x += v.x;
    s.y += v.y;
    s.z += v.z;
    s.w += v.w;
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

int ilog2_exact(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return ((1 << l) == v) ? l : -1;
}

template <typename T, int MODE, int WM, int WN, int TM, int TN>
const char* igemm_name() {
  static const std::string name = std::string("igemm_kernel<") + (sizeof(T) == 2 ? "bf16" : "f32") + "," +
                                  (MODE == kFwd ? "fwd" : MODE == kDgrad ? "dgrad" : "wgrad") + "," +
                                  std::to_string(WM * TM * 32) + "x" + std::to_string(WN * TN * 32) + ">";
  return name.c_str();
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
  return launch(ctx, igemm_kernel<T, MODE, WM, WN, TM, TN>, dim3(static_cast<unsigned>(wgs)), dim3(WM * WN * 64), a,
                igemm_name<T, MODE, WM, WN, TM, TN>(), flops, 0);
}

template <typename T, int MODE>
int launch_mode(Context* ctx, IgemmArgs& a, int tile_cfg, double flops) {
  switch (tile_cfg) {
    case 0:
      return launch_cfg<T, MODE, 2, 2, 2, 2>(ctx, a, flops);  // 128 x 128
    case 1:
      return launch_cfg<T, MODE, 2, 2, 2, 1>(ctx, a, flops);  // 128 x 64
    default:
      return launch_cfg<T, MODE, 2, 2, 1, 1>(ctx, a, flops);  // 64 x 64
  }
}

// 2 * N*Ho*Wo * K * R*S*C: the same for forward, data gradient and weight gradient;
// zero-padded input channels do no algorithmic work
double conv_flops(const ConvShape& s, int Ho, int Wo) {
  const int c = (s.c_logical > 0 && s.c_logical < s.C) ? s.c_logical : s.C;
  return 2.0 * s.N * Ho * Wo * static_cast<double>(s.K) * s.R * s.S * c;
}

int64_t tiles_for(int m, int n, int bm, int bn) {
  return static_cast<int64_t>((m + bm - 1) / bm) * ((n + bn - 1) / bn);
}

// Enough workgroups to give each of the 256 CUs some, with bigger tiles as
// soon as the problem can afford them.
int pick_tile(int gemm_m, int gemm_n, int splits) {
  if (gemm_n > 64 && tiles_for(gemm_m, gemm_n, 128, 128) * splits >= 384) return 0;
  if (tiles_for(gemm_m, gemm_n, 128, 64) * splits >= 384) return 1;
  return 2;
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

int conv2d_fwd(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* w, void* y, const void* add,
               const void* mask, const float* bias, int out_f32, int tile_cfg) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(x && w && y, "conv2d_fwd: null tensor");
  a.a_src = x;
  a.b_src = w;
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
  if (tile_cfg < 0) tile_cfg = pick_tile(a.gemm_m, a.gemm_n, 1);
  return dtype == kBF16 ? launch_mode<bf16, kFwd>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                        : launch_mode<float, kFwd>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
}

int conv2d_dgrad(Context* ctx, int dtype, const ConvShape& s, const void* dy, const void* w, void* dx, const void* add,
                 const void* mask, int tile_cfg) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(dy && w && dx, "conv2d_dgrad: null tensor");
  a.a_src = dy;
  a.b_src = w;
  a.out = dx;
  a.add = add;
  a.mask = mask;
  a.gemm_m = s.N * s.H * s.W;
  a.gemm_n = s.C;
  a.gemm_k = s.R * s.S * s.K;
  a.k_per_split = (a.gemm_k + 31) / 32 * 32;
  a.div_plane = FastDiv(s.H * s.W);
  a.div_width = FastDiv(s.W);
  if (tile_cfg < 0) tile_cfg = pick_tile(a.gemm_m, a.gemm_n, 1);
  return dtype == kBF16 ? launch_mode<bf16, kDgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                        : launch_mode<float, kDgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
}

int64_t conv2d_wgrad_workspace_bytes(const ConvShape& s, int dtype, int splits) {
  if (splits <= 1) return 0;
  (void)dtype;
  return static_cast<int64_t>(splits) * s.K * s.R * s.S * s.C * 4;
}

int conv2d_wgrad_pick_splits(const ConvShape& s, int dtype) {
  const int BK = dtype == kBF16 ? 32 : 16;
  int Ho, Wo;
  conv_output_hw(s, &Ho, &Wo);
  const int64_t pixels = static_cast<int64_t>(s.N) * Ho * Wo;
  const int gemm_m = s.K, gemm_n = s.R * s.S * s.C;
  int64_t tiles = tiles_for(gemm_m, gemm_n, 128, 128);
  if (tiles < 8) tiles = tiles_for(gemm_m, gemm_n, 64, 64);
  int64_t want = (768 + tiles - 1) / tiles;
  int64_t max_by_k = pixels / (4 * BK);  // at least four reduction steps per split
  if (max_by_k < 1) max_by_k = 1;
  if (want > max_by_k) want = max_by_k;
  if (want > 512) want = 512;
  if (want < 1) want = 1;
  return static_cast<int>(want);
}

int conv2d_wgrad(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* dy, float* dw, float* workspace,
                 int splits, int accumulate, int tile_cfg) {
  IgemmArgs a{};
  if (int rc = fill_common(a, s, dtype)) return rc;
  TCH_CHECK_ARG(x && dy && dw, "conv2d_wgrad: null tensor");
  TCH_CHECK_ARG(splits >= 1, "conv2d_wgrad: splits must be >= 1");
  TCH_CHECK_ARG(splits == 1 || workspace, "conv2d_wgrad: split reduction needs a workspace");
  const int BK = dtype == kBF16 ? 32 : 16;
  a.a_src = dy;
  a.b_src = x;
  a.gemm_m = s.K;
  a.gemm_n = s.R * s.S * s.C;
  a.gemm_k = s.N * a.Ho * a.Wo;
  int per = (a.gemm_k + splits - 1) / splits;
  per = (per + BK - 1) / BK * BK;
  splits = (a.gemm_k + per - 1) / per;  // drop empty tail splits
  a.splits = splits;
  a.k_per_split = per;
  a.accumulate = accumulate;
  a.out = splits > 1 ? static_cast<void*>(workspace) : static_cast<void*>(dw);
  a.div_plane = FastDiv(a.Ho * a.Wo);
  a.div_width = FastDiv(a.Wo);
  if (tile_cfg < 0) {
    tile_cfg = (a.gemm_m >= 128 && a.gemm_n >= 128 && tiles_for(a.gemm_m, a.gemm_n, 128, 128) * splits >= 256) ? 0 : 2;
  }
  int rc = dtype == kBF16 ? launch_mode<bf16, kWgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo))
                          : launch_mode<float, kWgrad>(ctx, a, tile_cfg, conv_flops(s, a.Ho, a.Wo));
  if (rc) return rc;
  if (splits > 1) {
    ReduceArgs r{workspace, dw, static_cast<int64_t>(a.gemm_m) * a.gemm_n, splits, accumulate};
    TCH_CHECK_ARG(r.n % 4 == 0, "conv2d_wgrad: filter size must be a multiple of 4");
    unsigned blocks = static_cast<unsigned>((r.n / 4 + 255) / 256);
    return launch(ctx, splitk_reduce_kernel, dim3(blocks), dim3(256), r, "splitk_reduce_kernel",
                  4.0 * r.n * (splits + 1 + (accumulate ? 1 : 0)), 1);
  }
  return 0;
}

}  // namespace tch
