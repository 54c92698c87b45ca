// Data movement of the Swin-B training step: cyclic shift + window partition (and its inverse, with the
// residual add), the 2x2 neighbourhood gather of patch merging (and its inverse), and the relative-position
// bias: table -> dense [heads, N, N] and the table's gradient from the attention-logit gradients.
// All HBM-bound gathers: every lane moves one 16-byte chunk of channels, so reads and writes are coalesced
// along the channel dimension whatever the permutation of tokens.
//
// Restated from the reference's readable statement of the model (train/swin_b_tiny.py): window_partition /
// window_reverse :8-19, torch.roll by -shift / +shift around them :116-131, the relative position index and
// the bias gather :35-59; patch merging and the shift mask are torchvision's (train/swin_b.py:38).
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

unsigned flat_blocks(int64_t items, int64_t cap = 16384) {
  int64_t b = (items + 255) / 256;
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return static_cast<unsigned>(b);
}

struct WindowArgs {
  const void* src;
  const void* add;  // optional, laid out like dst
  void* dst;
  int B, H, W, cc;  // cc = 16-byte chunks per token
  int ws, shift;
  int reverse;      // 0: image -> windows, 1: windows -> image
  int64_t chunks;   // B * H * W * cc
};

// window token t = (b, wh, ww, i, j) <-> pixel (b, (wh*ws + i + shift) mod H, (ww*ws + j + shift) mod W):
// roll by -shift, then partition.  Both directions are gathers indexed by the DESTINATION element.
__global__ __launch_bounds__(256) void window_kernel(WindowArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  const int nww = p.W / p.ws, nwh = p.H / p.ws;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < p.chunks; e += stride) {
    const int c = static_cast<int>(e % p.cc);
    int64_t t = e / p.cc;
    int64_t src_tok;
    if (!p.reverse) {
      // destination is a window token
      const int j = static_cast<int>(t % p.ws); t /= p.ws;
      const int i = static_cast<int>(t % p.ws); t /= p.ws;
      const int ww = static_cast<int>(t % nww); t /= nww;
      const int wh = static_cast<int>(t % nwh); t /= nwh;
      int h = wh * p.ws + i + p.shift, w = ww * p.ws + j + p.shift;
      if (h >= p.H) h -= p.H;
      if (w >= p.W) w -= p.W;
      src_tok = (t * p.H + h) * p.W + w;
    } else {
      // destination is a pixel
      const int w = static_cast<int>(t % p.W); t /= p.W;
      const int h = static_cast<int>(t % p.H); t /= p.H;
      int hs = h - p.shift, wsft = w - p.shift;
      if (hs < 0) hs += p.H;
      if (wsft < 0) wsft += p.W;
      const int wh = hs / p.ws, i = hs - wh * p.ws, ww = wsft / p.ws, j = wsft - ww * p.ws;
      src_tok = (((t * nwh + wh) * nww + ww) * p.ws + i) * p.ws + j;
    }
    static_cast<uint4*>(p.dst)[e] = static_cast<const uint4*>(p.src)[src_tok * p.cc + c];
  }
}

// the reverse direction with an addend needs arithmetic: typed variant
template <typename T>
__global__ __launch_bounds__(256) void window_reverse_add_kernel(WindowArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  const int nww = p.W / p.ws, nwh = p.H / p.ws;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < p.chunks; e += stride) {
    const int c = static_cast<int>(e % p.cc);
    int64_t t = e / p.cc;
    const int w = static_cast<int>(t % p.W); t /= p.W;
    const int h = static_cast<int>(t % p.H); t /= p.H;
    int hs = h - p.shift, wsft = w - p.shift;
    if (hs < 0) hs += p.H;
    if (wsft < 0) wsft += p.W;
    const int wh = hs / p.ws, i = hs - wh * p.ws, ww = wsft / p.ws, j = wsft - ww * p.ws;
    const int64_t src_tok = (((t * nwh + wh) * nww + ww) * p.ws + i) * p.ws + j;
    Chunk a, b;
    a.u = static_cast<const uint4*>(p.src)[src_tok * p.cc + c];
    b.u = static_cast<const uint4*>(p.add)[e];
    float va[E], vb[E];
    chunk_to_float<T>(a, va);
    chunk_to_float<T>(b, vb);
#pragma unroll
    for (int k = 0; k < E; ++k) va[k] += vb[k];
    static_cast<uint4*>(p.dst)[e] = float_to_chunk<T>(va).u;
  }
}

struct MergeArgs {
  const void* src;
  void* dst;
  int B, H, W, cc;  // the UNMERGED image: [B, H, W, C]; merged: [B, H/2, W/2, 4C]
  int reverse;      // 0: image -> merged, 1: merged -> image
  int64_t chunks;   // B * H * W * cc (same count both ways)
};

// merged[b, h2, w2, q*C + c] = image[b, 2*h2 + (q & 1), 2*w2 + (q >> 1), c]: the concatenation order
// x0 = (even row, even col), x1 = (odd, even), x2 = (even, odd), x3 = (odd, odd)
__global__ __launch_bounds__(256) void patch_merge_kernel(MergeArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  // odd sizes: the image is padded with a zero row / column (the merged map is (H + 1) / 2 x (W + 1) / 2)
  const int H2 = (p.H + 1) / 2, W2 = (p.W + 1) / 2;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < p.chunks; e += stride) {
    int64_t src;
    bool real = true;
    if (!p.reverse) {
      const int c = static_cast<int>(e % p.cc);
      int64_t t = e / p.cc;
      const int q = static_cast<int>(t % 4); t /= 4;
      const int w2 = static_cast<int>(t % W2); t /= W2;
      const int h2 = static_cast<int>(t % H2); t /= H2;
      const int h = 2 * h2 + (q & 1), w = 2 * w2 + (q >> 1);
      real = h < p.H && w < p.W;
      src = (((t * p.H + h) * p.W + w) * p.cc) + c;
    } else {
      const int c = static_cast<int>(e % p.cc);
      int64_t t = e / p.cc;
      const int w = static_cast<int>(t % p.W); t /= p.W;
      const int h = static_cast<int>(t % p.H); t /= p.H;
      const int q = (h & 1) + 2 * (w & 1);
      src = ((((t * H2 + (h >> 1)) * W2 + (w >> 1)) * 4 + q) * p.cc) + c;
    }
    static_cast<uint4*>(p.dst)[e] = real ? static_cast<const uint4*>(p.src)[src] : make_uint4(0u, 0u, 0u, 0u);
  }
}

struct RelPosArgs {
  const float* table;    // [entries][heads]
  const int32_t* index;  // [N*N]
  float* bias;           // [heads][N*N]
  const float* dbias;    // [heads][N*N]   (backward)
  float* dtable;         // [entries][heads] (backward, (+)=)
  int heads, nn, entries, accumulate;
};

__global__ __launch_bounds__(256) void relpos_gather_kernel(RelPosArgs p) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= p.heads * p.nn) return;
  const int h = e / p.nn, ij = e - h * p.nn;
  const int idx = p.index[ij];
  p.bias[e] = idx < 0 ? -INFINITY : p.table[idx * p.heads + h];   // a negative index marks padding: masked out
}

// the same for up to kRelPosBatch bias tables in one launch: blockIdx.y names the table
constexpr int kRelPosBatch = 8;
struct RelPosBatchArgs {
  const float* table[kRelPosBatch];    // [entries][heads[k]]
  const int32_t* index[kRelPosBatch];  // [nn]
  float* bias[kRelPosBatch];           // [heads[k]][nn]
  int heads[kRelPosBatch];
  int nn;
};

__global__ __launch_bounds__(256) void relpos_gather_batch_kernel(RelPosBatchArgs p) {
  const int k = blockIdx.y;
  const int heads = p.heads[k];
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= heads * p.nn) return;
  const int h = e / p.nn, ij = e - h * p.nn;
  const int idx = p.index[k][ij];
  p.bias[k][e] = idx < 0 ? -INFINITY : p.table[k][idx * heads + h];
}

// one wavefront per (table entry, head): the (i, j) pairs that point at the entry are summed in index order
__global__ __launch_bounds__(64) void relpos_scatter_kernel(RelPosArgs p) {
  const int entry = blockIdx.x / p.heads, h = blockIdx.x - entry * p.heads;
  float s = 0.f;
  for (int ij = threadIdx.x; ij < p.nn; ij += 64)
    if (p.index[ij] == entry) s += p.dbias[h * p.nn + ij];
  s = wave_sum(s);
  if (threadIdx.x == 0) {
    float* dst = p.dtable + entry * p.heads + h;
    *dst = p.accumulate ? *dst + s : s;
  }
}

// the same from a precomputed inverse of the index: entry e receives the pairs list[ptr[e] .. ptr[e+1]), summed
// by one wavefront per (entry, head) in a fixed order
struct RelPosCsrArgs {
  const float* dbias;    // [heads][pairs]
  const int32_t* ptr;    // [entries + 1]
  const int32_t* list;   // [ptr[entries]] pair numbers
  float* dtable;         // [entries][heads]
  int heads, pairs, entries, accumulate;
};

__global__ __launch_bounds__(256) void relpos_scatter_csr_kernel(RelPosCsrArgs p) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= p.entries * p.heads) return;
  const int entry = t / p.heads, h = t - entry * p.heads;
  const int end = p.ptr[entry + 1];
  float s = 0.f;
  for (int i = p.ptr[entry] + lane; i < end; i += 64) s += p.dbias[static_cast<int64_t>(h) * p.pairs + p.list[i]];
  s = wave_sum(s);
  if (lane == 0) {
    float* dst = p.dtable + t;
    *dst = p.accumulate ? *dst + s : s;
  }
}

struct ColSumArgs {
  const void* x;   // [rows][cols], T
  float* partial;  // [slabs][cols]
  float* out;      // [cols] (second pass)
  int rows, cols, rows_per_slab, slabs, accumulate;
};

// sum over the rows of a matrix whose width need not be a multiple of a chunk: one thread per column
template <typename T>
__global__ __launch_bounds__(256) void col_sum_rows_kernel(ColSumArgs p) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= p.cols) return;
  const int r0 = blockIdx.y * p.rows_per_slab;
  const int r1 = r0 + p.rows_per_slab < p.rows ? r0 + p.rows_per_slab : p.rows;
  const T* src = static_cast<const T*>(p.x) + c;
  float s = 0.f;
  for (int r = r0; r < r1; ++r) s += Elem<T>::load(src + static_cast<int64_t>(r) * p.cols);
  p.partial[static_cast<int64_t>(blockIdx.y) * p.cols + c] = s;
}

__global__ __launch_bounds__(256) void col_sum_slabs_kernel(ColSumArgs p) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= p.cols) return;
  float s = 0.f;
  for (int k = 0; k < p.slabs; ++k) s += p.partial[static_cast<int64_t>(k) * p.cols + c];
  p.out[c] = p.accumulate ? p.out[c] + s : s;
}

}  // namespace

int window_partition(Context* ctx, int dtype, const void* src, void* dst, const void* add, int B, int H, int W, int C,
                     int window, int shift, int reverse) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "window_partition: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(src && dst && B > 0 && C > 0 && C % E == 0, "window_partition: bad tensor arguments");
  TCH_CHECK_ARG(window > 0 && H % window == 0 && W % window == 0, "window_partition: the window must tile the image");
  TCH_CHECK_ARG(shift >= 0 && shift < window, "window_partition: shift must be in [0, window)");
  TCH_CHECK_ARG(!add || reverse, "window_partition: the addend goes with the reverse direction");
  WindowArgs a{src, add, dst, B, H, W, C / E, window, shift, reverse, static_cast<int64_t>(B) * H * W * (C / E)};
  const double bytes = static_cast<double>(a.chunks) * 16.0 * (add ? 3.0 : 2.0);
  const dim3 grid(flat_blocks(a.chunks));
  if (add)
    return dtype == kBF16 ? launch(ctx, window_reverse_add_kernel<bf16>, grid, dim3(256), a, "window_reverse_add_kernel<bf16>", bytes, 1)
                          : launch(ctx, window_reverse_add_kernel<float>, grid, dim3(256), a, "window_reverse_add_kernel<f32>", bytes, 1);
  return launch(ctx, window_kernel, grid, dim3(256), a, reverse ? "window_kernel<reverse>" : "window_kernel<partition>", bytes, 1);
}

int patch_merge_gather(Context* ctx, int dtype, const void* src, void* dst, int B, int H, int W, int C, int reverse) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "patch_merge_gather: dtype must be f32(0) or bf16(1)");
  const int E = dtype == kBF16 ? 8 : 4;
  TCH_CHECK_ARG(src && dst && B > 0 && C > 0 && C % E == 0 && H > 0 && W > 0,
                "patch_merge_gather: bad arguments (C a multiple of a 16-byte chunk)");
  // one thread per 16-byte chunk of the destination: the merged map (padded to even sides) forward, the image backward
  const int64_t dst_pixels = reverse ? static_cast<int64_t>(H) * W : static_cast<int64_t>((H + 1) / 2) * ((W + 1) / 2) * 4;
  MergeArgs a{src, dst, B, H, W, C / E, reverse, B * dst_pixels * (C / E)};
  return launch(ctx, patch_merge_kernel, dim3(flat_blocks(a.chunks)), dim3(256), a,
                reverse ? "patch_merge_kernel<reverse>" : "patch_merge_kernel<gather>", static_cast<double>(a.chunks) * 32.0, 1);
}

int relpos_bias_gather(Context* ctx, const float* table, const int32_t* index, float* bias, int heads, int tokens,
                       int entries) {
  TCH_CHECK_ARG(table && index && bias && heads > 0 && tokens > 0 && entries > 0, "relpos_bias_gather: bad arguments");
  RelPosArgs a{table, index, bias, nullptr, nullptr, heads, tokens * tokens, entries, 0};
  return launch(ctx, relpos_gather_kernel, dim3((heads * a.nn + 255) / 256), dim3(256), a, "relpos_gather_kernel",
                8.0 * heads * a.nn, 1);
}

int relpos_bias_scatter(Context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads, int tokens,
                        int entries, int accumulate) {
  TCH_CHECK_ARG(dbias && index && dtable && heads > 0 && tokens > 0 && entries > 0, "relpos_bias_scatter: bad arguments");
  RelPosArgs a{nullptr, index, nullptr, dbias, dtable, heads, tokens * tokens, entries, accumulate};
  return launch(ctx, relpos_scatter_kernel, dim3(entries * heads), dim3(64), a, "relpos_scatter_kernel",
                4.0 * entries * heads * a.nn, 1);
}

int relpos_bias_gather_pairs(Context* ctx, const float* table, const int32_t* index, float* bias, int heads, int pairs,
                             int entries) {
  TCH_CHECK_ARG(table && index && bias && heads > 0 && pairs > 0 && entries > 0, "relpos_bias_gather_pairs: bad arguments");
  RelPosArgs a{table, index, bias, nullptr, nullptr, heads, pairs, entries, 0};
  return launch(ctx, relpos_gather_kernel, dim3((heads * a.nn + 255) / 256), dim3(256), a, "relpos_gather_kernel",
                8.0 * heads * a.nn, 1);
}

int relpos_bias_gather_batch(Context* ctx, const float* const* tables, const int32_t* const* indices, float* const* biases,
                             const int* heads, int count, int pairs, int entries) {
  TCH_CHECK_ARG(tables && indices && biases && heads && count > 0 && pairs > 0 && entries > 0,
                "relpos_bias_gather_batch: bad arguments");
  for (int k = 0; k < count; ++k)
    TCH_CHECK_ARG(tables[k] && indices[k] && biases[k] && heads[k] > 0, "relpos_bias_gather_batch: bad table in the batch");
  for (int first = 0; first < count; first += kRelPosBatch) {
    const int n = count - first < kRelPosBatch ? count - first : kRelPosBatch;
    RelPosBatchArgs a{};
    int most = 0, total = 0;
    for (int k = 0; k < n; ++k) {
      a.table[k] = tables[first + k];
      a.index[k] = indices[first + k];
      a.bias[k] = biases[first + k];
      a.heads[k] = heads[first + k];
      most = a.heads[k] > most ? a.heads[k] : most;
      total += a.heads[k];
    }
    a.nn = pairs;
    const int rc = launch(ctx, relpos_gather_batch_kernel, dim3((most * pairs + 255) / 256, n), dim3(256), a,
                          "relpos_gather_batch_kernel", 8.0 * total * pairs, 1);
    if (rc != 0) return rc;
  }
  return 0;
}

int relpos_bias_scatter_pairs(Context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads, int pairs,
                              int entries, int accumulate) {
  TCH_CHECK_ARG(dbias && index && dtable && heads > 0 && pairs > 0 && entries > 0, "relpos_bias_scatter_pairs: bad arguments");
  RelPosArgs a{nullptr, index, nullptr, dbias, dtable, heads, pairs, entries, accumulate};
  return launch(ctx, relpos_scatter_kernel, dim3(entries * heads), dim3(64), a, "relpos_scatter_kernel",
                4.0 * entries * heads * a.nn, 1);
}

int relpos_bias_scatter_csr(Context* ctx, const float* dbias, const int32_t* ptr, const int32_t* list, float* dtable,
                            int heads, int pairs, int entries, int accumulate) {
  TCH_CHECK_ARG(dbias && ptr && list && dtable && heads > 0 && pairs > 0 && entries > 0, "relpos_bias_scatter_csr: bad arguments");
  RelPosCsrArgs a{dbias, ptr, list, dtable, heads, pairs, entries, accumulate};
  return launch(ctx, relpos_scatter_csr_kernel, dim3((entries * heads + 3) / 4), dim3(256), a,
                "relpos_scatter_csr_kernel", 8.0 * heads * pairs, 1);
}

int64_t column_sum_workspace_floats(int rows, int cols) {
  int slabs = rows / 64;
  if (slabs > 32) slabs = 32;
  if (slabs < 1) slabs = 1;
  return static_cast<int64_t>(slabs) * cols;
}

int column_sum(Context* ctx, int dtype, const void* x, float* out, int rows, int cols, int accumulate, float* workspace) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "column_sum: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(x && out && workspace && rows > 0 && cols > 0, "column_sum: bad arguments");
  int slabs = static_cast<int>(column_sum_workspace_floats(rows, cols) / cols);
  ColSumArgs a{x, workspace, out, rows, cols, (rows + slabs - 1) / slabs, slabs, accumulate};
  a.slabs = (rows + a.rows_per_slab - 1) / a.rows_per_slab;
  const dim3 grid((cols + 255) / 256, a.slabs);
  const double bytes = static_cast<double>(rows) * cols * (dtype == kBF16 ? 2.0 : 4.0);
  int rc = dtype == kBF16 ? launch(ctx, col_sum_rows_kernel<bf16>, grid, dim3(256), a, "col_sum_rows_kernel<bf16>", bytes, 1)
                          : launch(ctx, col_sum_rows_kernel<float>, grid, dim3(256), a, "col_sum_rows_kernel<f32>", bytes, 1);
  if (rc) return rc;
  return launch(ctx, col_sum_slabs_kernel, dim3((cols + 255) / 256), dim3(256), a, "col_sum_slabs_kernel",
                4.0 * a.slabs * cols, 1);
}

}  // namespace tch
