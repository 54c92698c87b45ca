// Fused softmax-cross-entropy (forward + gradient in one pass over the
// logits), fused SGD-momentum over a flat fp32 parameter buffer with a bf16
// shadow copy, the micro-batch gradient accumulator, and small helpers.
// All HBM-bound.
//
// Restated arithmetic and its reference call sites:
//   nn.CrossEntropyLoss (mean)              train/swin_b.py:42, train/resnet152.py:26
//   loss /= global_batch / batch            pytorch/torch_col/dynamic_batch.py:112-120
//   torch.optim.SGD(momentum, weight_decay) train/resnet152.py:27-28,
//     with momentum buffers pre-zeroed      pytorch/torch_col/util.py:182-191
//   GradAccumulator.accumulate              pytorch/torch_col/accumulate.py:20-24
#include "kernels.h"
#include "ops.h"

namespace tch {
namespace {

struct CeArgs {
  const float* logits;
  const int64_t* labels;
  float* loss_rows;
  void* dlogits;
  int rows, classes, ld;
  float grad_scale;  // d(loss_mean * loss_scale)/d(loss_row) = loss_scale / rows
};

// one wavefront per row
template <typename T>
__global__ __launch_bounds__(64) void softmax_ce_kernel(CeArgs p) {
  const int row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = p.logits + static_cast<int64_t>(row) * p.classes;
  float mx = -INFINITY;
  for (int c = lane; c < p.classes; c += 64) mx = fmaxf(mx, z[c]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int c = lane; c < p.classes; c += 64) sum += expf(z[c] - mx);
  sum = wave_sum(sum);
  const float lse = mx + logf(sum);
  const int label = static_cast<int>(p.labels[row]);
  if (lane == 0) p.loss_rows[row] = lse - z[label];
  T* g = static_cast<T*>(p.dlogits) + static_cast<int64_t>(row) * p.ld;
  const float inv = 1.f / sum;
  for (int c = lane; c < p.classes; c += 64) {
    float sm = expf(z[c] - mx) * inv;
    Elem<T>::store(g + c, (sm - (c == label ? 1.f : 0.f)) * p.grad_scale);
  }
}

// Language-model form: one workgroup per row (vocabulary-sized rows), logits with their own leading
// dimension, rows whose label is negative are ignored (zero loss, zero gradient).
struct CeWideArgs {
  const float* logits;
  const int64_t* labels;
  float* loss_rows;
  void* dlogits;
  int rows, classes, ld_logits, ld_dlogits;
  float grad_scale;
};

__device__ inline float block_reduce(float v, bool take_max, float* scratch) {
  v = take_max ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // scratch may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) r = take_max ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_ce_wide_kernel(CeWideArgs p) {
  __shared__ float scratch[4];
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* z = p.logits + static_cast<int64_t>(row) * p.ld_logits;
  T* g = static_cast<T*>(p.dlogits) + static_cast<int64_t>(row) * p.ld_dlogits;
  const int64_t label = p.labels[row];
  if (label < 0 || label >= p.classes) {
    if (tid == 0) p.loss_rows[row] = 0.f;
    for (int c = tid; c < p.classes; c += 256) Elem<T>::store(g + c, 0.f);
    return;
  }
  float mx = -INFINITY;
  for (int c = tid; c < p.classes; c += 256) mx = fmaxf(mx, z[c]);
  mx = block_reduce(mx, true, scratch);
  float sum = 0.f;
  for (int c = tid; c < p.classes; c += 256) sum += expf(z[c] - mx);
  sum = block_reduce(sum, false, scratch);
  if (tid == 0) p.loss_rows[row] = mx + logf(sum) - z[label];
  const float inv = 1.f / sum;
  for (int c = tid; c < p.classes; c += 256) {
    const float sm = expf(z[c] - mx) * inv;
    Elem<T>::store(g + c, (sm - (c == label ? 1.f : 0.f)) * p.grad_scale);
  }
}

// The same with the whole row held in registers: 1024 threads keep up to 16 four-float pieces each (rows up
// to 65536 classes), so the logits are read once and the gradient written once.  Needs 16-byte aligned rows
// on both sides and room for the last piece (the columns between `classes` and the next multiple of four
// receive zeros).
constexpr int kRowPieces = 16;

__device__ inline float block_reduce_1024(float v, bool take_max, float* scratch) {
  v = take_max ? wave_max(v) : wave_sum(v);
  __syncthreads();   // the previous reduction's readers are done
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) r = take_max ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}

template <typename T>
__global__ __launch_bounds__(1024) void softmax_ce_row_kernel(CeWideArgs p) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float4* z = reinterpret_cast<const float4*>(p.logits + static_cast<int64_t>(row) * p.ld_logits);
  T* g = static_cast<T*>(p.dlogits) + static_cast<int64_t>(row) * p.ld_dlogits;
  const int pieces = (p.classes + 3) >> 2;
  const int64_t label = p.labels[row];
  const bool ignored = label < 0 || label >= p.classes;
  float v[kRowPieces][4];
  float mx = -INFINITY;
  if (!ignored) {
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i) {
      const int pc = tid + 1024 * i;
      if (pc < pieces) {
        const float4 t = z[pc];
        v[i][0] = t.x;
        v[i][1] = t.y;
        v[i][2] = t.z;
        v[i][3] = t.w;
        if (pc == pieces - 1) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (pc * 4 + e >= p.classes) v[i][e] = -INFINITY;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[i][e] = -INFINITY;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) mx = fmaxf(mx, v[i][e]);
    }
  }
  mx = block_reduce_1024(mx, true, scratch);
  float sum = 0.f;
  if (!ignored) {
#pragma unroll
    for (int i = 0; i < kRowPieces; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[i][e] = __expf(v[i][e] - mx);
        sum += v[i][e];
      }
  }
  sum = block_reduce_1024(sum, false, scratch);
  if (tid == 0) p.loss_rows[row] = ignored ? 0.f : mx + logf(sum) - p.logits[static_cast<int64_t>(row) * p.ld_logits + label];
  const float mul = ignored ? 0.f : p.grad_scale / sum;
#pragma unroll
  for (int i = 0; i < kRowPieces; ++i) {
    const int pc = tid + 1024 * i;
    if (pc >= pieces) continue;
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = ignored ? 0.f : v[i][e] * mul;
      if (pc * 4 + e == label) o[e] -= p.grad_scale;
    }
    if constexpr (sizeof(T) == 2) {
      uint2 w;
      w.x = float_to_bf16_bits(o[0]) | (static_cast<uint32_t>(float_to_bf16_bits(o[1])) << 16);
      w.y = float_to_bf16_bits(o[2]) | (static_cast<uint32_t>(float_to_bf16_bits(o[3])) << 16);
      *reinterpret_cast<uint2*>(g + pc * 4) = w;
    } else {
      *reinterpret_cast<float4*>(g + pc * 4) = make_float4(o[0], o[1], o[2], o[3]);
    }
  }
}

struct MeanArgs {
  const float* in;
  float* out;
  int n;
  float divisor;
};

// one workgroup of 1024 threads: thread t adds rows t, t + 1024, ...; the wavefronts' sums meet in LDS in wavefront
// order (a fixed order: the mean does not change from run to run)
__global__ __launch_bounds__(1024) void mean_kernel(MeanArgs p) {
  __shared__ float part[16];
  float s = 0.f;
  for (int i = threadIdx.x; i < p.n; i += 1024) s += p.in[i];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) t += part[w];
    *p.out = t / p.divisor;
  }
}

struct SgdArgs {
  float* param;
  const float* grad;
  float* buf;
  uint16_t* shadow;
  int64_t n;
  float lr, momentum, wd;
  int aligned;   // every buffer starts on a 16-byte boundary (the shadow on 8): 16-byte accesses are in order
};

__global__ __launch_bounds__(256) void sgd_kernel(SgdArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; i < p.n; i += stride) {
    if (p.aligned && i + 4 <= p.n) {
      float4 w = load_streaming_f4(p.param + i);
      float4 g = load_streaming_f4(p.grad + i);
      float4 b = load_streaming_f4(p.buf + i);
      b.x = p.momentum * b.x + (g.x + p.wd * w.x);
      b.y = p.momentum * b.y + (g.y + p.wd * w.y);
      b.z = p.momentum * b.z + (g.z + p.wd * w.z);
      b.w = p.momentum * b.w + (g.w + p.wd * w.w);
      w.x -= p.lr * b.x;
      w.y -= p.lr * b.y;
      w.z -= p.lr * b.z;
      w.w -= p.lr * b.w;
      store_streaming_f4(p.param + i, w);
      store_streaming_f4(p.buf + i, b);
      if (p.shadow) {
        uint2 s;
        s.x = float_to_bf16_bits(w.x) | (static_cast<uint32_t>(float_to_bf16_bits(w.y)) << 16);
        s.y = float_to_bf16_bits(w.z) | (static_cast<uint32_t>(float_to_bf16_bits(w.w)) << 16);
        *reinterpret_cast<uint2*>(p.shadow + i) = s;
      }
    } else {
      for (int64_t j = i; j < p.n && j < i + 4; ++j) {
        float w = p.param[j];
        float b = p.momentum * p.buf[j] + (p.grad[j] + p.wd * w);
        w -= p.lr * b;
        p.param[j] = w;
        p.buf[j] = b;
        if (p.shadow) p.shadow[j] = float_to_bf16_bits(w);
      }
    }
  }
}

struct AccumArgs {
  float* global;
  float* grad;
  int64_t n;
};

// global += grad; grad = 0
__global__ __launch_bounds__(256) void accumulate_kernel(AccumArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; i < p.n; i += stride) {
    if (i + 4 <= p.n) {
      float4 a = *reinterpret_cast<float4*>(p.global + i);
      float4 g = *reinterpret_cast<float4*>(p.grad + i);
      a.x += g.x;
      a.y += g.y;
      a.z += g.z;
      a.w += g.w;
      *reinterpret_cast<float4*>(p.global + i) = a;
      *reinterpret_cast<float4*>(p.grad + i) = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      for (int64_t j = i; j < p.n; ++j) {
        p.global[j] += p.grad[j];
        p.grad[j] = 0.f;
      }
    }
  }
}

struct FillArgs {
  uint32_t* ptr;
  int64_t words;
};

__global__ __launch_bounds__(256) void fill_zero_kernel(FillArgs p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < p.words; i += stride) p.ptr[i] = 0u;
}

struct BiasGradArgs {
  const void* dy;
  float* dbias;
  int rows, cols, ld, accumulate;
  float* partial;     // tall form with row slabs: [slabs][cols] partial sums instead of dbias
  int rows_per_slab;  // tall form: rows one workgroup (blockIdx.y) covers
};

// one lane per column; rows are few (the batch)
template <typename T>
__global__ __launch_bounds__(256) void bias_grad_kernel(BiasGradArgs p) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= p.cols) return;
  float s = 0.f;
  const T* src = static_cast<const T*>(p.dy) + c;
  for (int r = 0; r < p.rows; ++r) s += Elem<T>::load(src + static_cast<int64_t>(r) * p.ld);
  p.dbias[c] = p.accumulate ? p.dbias[c] + s : s;
}

// many rows (tokens): 8 chunk columns x 32 row lanes per workgroup, 16-byte loads, the row lanes
// meet in LDS in a fixed order
template <typename T>
__global__ __launch_bounds__(256) void bias_grad_tall_kernel(BiasGradArgs p) {
  constexpr int E = Elem<T>::kPerChunk;
  __shared__ float red[32][8 * E + 1];
  const int tx = threadIdx.x & 7, ty = threadIdx.x >> 3;
  const int col = (blockIdx.x * 8 + tx) * E;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = 0.f;
  const int r_begin = blockIdx.y * p.rows_per_slab;
  const int r_end = r_begin + p.rows_per_slab < p.rows ? r_begin + p.rows_per_slab : p.rows;
  if (col < p.cols) {
    const T* src = static_cast<const T*>(p.dy) + col;
    for (int r = r_begin + ty; r < r_end; r += 32) {
      Chunk c;
      c.u = *reinterpret_cast<const uint4*>(src + static_cast<int64_t>(r) * p.ld);
      float v[E];
      chunk_to_float<T>(c, v);
#pragma unroll
      for (int e = 0; e < E; ++e) s[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) red[ty][tx * E + e] = s[e];
  __syncthreads();
  if (threadIdx.x < 8 * E) {
    const int c = blockIdx.x * 8 * E + threadIdx.x;
    if (c < p.cols) {
      float t = 0.f;
      for (int y = 0; y < 32; ++y) t += red[y][threadIdx.x];
      if (p.partial)
        p.partial[static_cast<int64_t>(blockIdx.y) * p.cols + c] = t;
      else
        p.dbias[c] = p.accumulate ? p.dbias[c] + t : t;
    }
  }
}

struct SlabSumArgs {
  const float* partial;  // [slabs][cols]
  float* out;
  int slabs, cols, accumulate;
};

__global__ __launch_bounds__(256) void slab_sum_kernel(SlabSumArgs p) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= p.cols) return;
  float t = 0.f;
  for (int s = 0; s < p.slabs; ++s) t += p.partial[static_cast<int64_t>(s) * p.cols + c];
  p.out[c] = p.accumulate ? p.out[c] + t : t;
}

unsigned flat_blocks(int64_t n_vec) {
  int64_t b = (n_vec + 255) / 256;
  if (b > (1 << 20)) b = 1 << 20;
  if (b < 1) b = 1;
  return static_cast<unsigned>(b);
}

}  // namespace

int softmax_ce_fwd_bwd(Context* ctx, int dtype, const float* logits, const int64_t* labels, float* loss_rows,
                       float* loss_mean, void* dlogits, int rows, int classes, int ld_dlogits, float grad_scale) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "softmax_ce: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(logits && labels && loss_rows && loss_mean && dlogits, "softmax_ce: null tensor");
  TCH_CHECK_ARG(rows > 0 && classes > 0 && ld_dlogits >= classes, "softmax_ce: bad shape");
  CeArgs a{logits, labels, loss_rows, dlogits, rows, classes, ld_dlogits, grad_scale};
  const double bytes = static_cast<double>(rows) * classes * (4.0 + (dtype == kBF16 ? 2.0 : 4.0));
  int rc = dtype == kBF16 ? launch(ctx, softmax_ce_kernel<bf16>, dim3(rows), dim3(64), a, "softmax_ce_kernel<bf16>", bytes, 1)
                          : launch(ctx, softmax_ce_kernel<float>, dim3(rows), dim3(64), a, "softmax_ce_kernel<f32>", bytes, 1);
  if (rc) return rc;
  MeanArgs m{loss_rows, loss_mean, rows, static_cast<float>(rows)};
  return launch(ctx, mean_kernel, dim3(1), dim3(1024), m, "mean_kernel", 4.0 * rows, 1);
}

int softmax_ce_lm(Context* ctx, int dtype, const float* logits, int ld_logits, const int64_t* labels, float* loss_rows,
                  float* loss_mean, void* dlogits, int ld_dlogits, int rows, int classes, int valid_rows,
                  float loss_scale) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "softmax_ce_lm: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(logits && labels && loss_rows && loss_mean && dlogits, "softmax_ce_lm: null tensor");
  TCH_CHECK_ARG(rows > 0 && classes > 0 && ld_logits >= classes && ld_dlogits >= classes && valid_rows > 0 &&
                    valid_rows <= rows,
                "softmax_ce_lm: bad shape");
  CeWideArgs a{logits, labels, loss_rows, dlogits, rows, classes, ld_logits, ld_dlogits,
               loss_scale / static_cast<float>(valid_rows)};
  const double bytes = static_cast<double>(rows) * classes * (4.0 + (dtype == kBF16 ? 2.0 : 4.0));
  const int padded = (classes + 3) / 4 * 4;
  const int eb = dtype == kBF16 ? 2 : 4;
  const bool in_registers = padded <= kRowPieces * 4096 && padded <= ld_logits && padded <= ld_dlogits && ld_logits % 4 == 0 &&
                            (static_cast<int64_t>(ld_dlogits) * eb) % 16 == 0 &&
                            (reinterpret_cast<uintptr_t>(logits) & 15) == 0 && (reinterpret_cast<uintptr_t>(dlogits) & 15) == 0;
  int rc;
  if (in_registers) {
    rc = dtype == kBF16
             ? launch(ctx, softmax_ce_row_kernel<bf16>, dim3(rows), dim3(1024), a, "softmax_ce_row_kernel<bf16>", bytes, 1)
             : launch(ctx, softmax_ce_row_kernel<float>, dim3(rows), dim3(1024), a, "softmax_ce_row_kernel<f32>", bytes, 1);
  } else {
    rc = dtype == kBF16
             ? launch(ctx, softmax_ce_wide_kernel<bf16>, dim3(rows), dim3(256), a, "softmax_ce_wide_kernel<bf16>", bytes, 1)
             : launch(ctx, softmax_ce_wide_kernel<float>, dim3(rows), dim3(256), a, "softmax_ce_wide_kernel<f32>", bytes, 1);
  }
  if (rc) return rc;
  MeanArgs m{loss_rows, loss_mean, rows, static_cast<float>(valid_rows)};
  return launch(ctx, mean_kernel, dim3(1), dim3(1024), m, "mean_kernel", 4.0 * rows, 1);
}

int sgd_momentum_step(Context* ctx, float* param, const float* grad, float* momentum_buf, void* shadow_bf16,
                      int64_t n, float lr, float momentum, float weight_decay) {
  TCH_CHECK_ARG(param && grad && momentum_buf && n > 0, "sgd_momentum_step: null tensor or empty");
  SgdArgs a{param, grad, momentum_buf, static_cast<uint16_t*>(shadow_bf16), n, lr, momentum, weight_decay, 0};
  a.aligned = ((reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(grad) | reinterpret_cast<uintptr_t>(momentum_buf)) & 15) == 0 &&
              (reinterpret_cast<uintptr_t>(shadow_bf16) & 7) == 0;
  return launch(ctx, sgd_kernel, dim3(flat_blocks((n + 3) / 4)), dim3(256), a, "sgd_kernel",
                static_cast<double>(n) * (shadow_bf16 ? 22.0 : 20.0), 1);
}

int grad_accumulate(Context* ctx, float* global, float* grad, int64_t n) {
  TCH_CHECK_ARG(global && grad && n > 0, "grad_accumulate: null tensor or empty");
  AccumArgs a{global, grad, n};
  return launch(ctx, accumulate_kernel, dim3(flat_blocks((n + 3) / 4)), dim3(256), a, "accumulate_kernel",
                static_cast<double>(n) * 16.0, 1);
}

int fill_zero(Context* ctx, void* ptr, int64_t bytes) {
  TCH_CHECK_ARG(ptr && bytes > 0 && bytes % 4 == 0, "fill_zero: size must be a positive multiple of 4 bytes");
  FillArgs a{static_cast<uint32_t*>(ptr), bytes / 4};
  return launch(ctx, fill_zero_kernel, dim3(flat_blocks(a.words)), dim3(256), a, "fill_zero_kernel",
                static_cast<double>(bytes), 1);
}

int bias_grad(Context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld, int accumulate,
              float* workspace, int64_t workspace_floats) {
  TCH_CHECK_ARG(dtype == kBF16 || dtype == kF32, "bias_grad: dtype must be f32(0) or bf16(1)");
  TCH_CHECK_ARG(dy && dbias && rows > 0 && cols > 0 && ld >= cols, "bias_grad: bad arguments");
  BiasGradArgs a{dy, dbias, rows, cols, ld, accumulate, nullptr, rows};
  const double bytes = static_cast<double>(rows) * cols * (dtype == kBF16 ? 2.0 : 4.0);
  const int E = dtype == kBF16 ? 8 : 4;
  if (rows >= 32 && cols % E == 0 && ld % E == 0 && (reinterpret_cast<uintptr_t>(dy) & 15) == 0) {
    // with scratch memory the rows are cut into slabs (more workgroups), summed by a second small launch
    int slabs = 1;
    if (workspace) {
      slabs = rows / 256;
      if (slabs > 64) slabs = 64;
      if (static_cast<int64_t>(slabs) * cols > workspace_floats) slabs = static_cast<int>(workspace_floats / cols);
      if (slabs < 1) slabs = 1;
    }
    if (slabs > 1) {
      a.partial = workspace;
      a.rows_per_slab = (rows + slabs - 1) / slabs;
      slabs = (rows + a.rows_per_slab - 1) / a.rows_per_slab;
    }
    const dim3 grid((cols / E + 7) / 8, slabs);
    int rc = dtype == kBF16
                 ? launch(ctx, bias_grad_tall_kernel<bf16>, grid, dim3(256), a, "bias_grad_tall_kernel<bf16>", bytes, 1)
                 : launch(ctx, bias_grad_tall_kernel<float>, grid, dim3(256), a, "bias_grad_tall_kernel<f32>", bytes, 1);
    if (rc || slabs == 1) return rc;
    SlabSumArgs s{workspace, dbias, slabs, cols, accumulate};
    return launch(ctx, slab_sum_kernel, dim3((cols + 255) / 256), dim3(256), s, "slab_sum_kernel", 4.0 * slabs * cols, 1);
  }
  return dtype == kBF16 ? launch(ctx, bias_grad_kernel<bf16>, dim3((cols + 255) / 256), dim3(256), a, "bias_grad_kernel<bf16>", bytes, 1)
                        : launch(ctx, bias_grad_kernel<float>, dim3((cols + 255) / 256), dim3(256), a, "bias_grad_kernel<f32>", bytes, 1);
}

}  // namespace tch
