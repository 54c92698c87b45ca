// Shared device-side helpers and the host-side launch plumbing for the HIP
// kernels of the colocated training step (gfx950 / CDNA4 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <type_traits>

namespace tch {

// ---------------------------------------------------------------------------
// element types
// ---------------------------------------------------------------------------

// bf16 is kept as raw bits in memory; arithmetic is always done in fp32.
struct bf16 {
  uint16_t v;
};

enum DType : int { kF32 = 0, kBF16 = 1 };

__host__ __device__ inline float bf16_bits_to_float(uint16_t b) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = static_cast<uint32_t>(b) << 16;
  return c.f;
}

// round-to-nearest-even, NaN stays NaN (quiet bit forced); on the device this is the hardware conversion
// (v_cvt_pk_bf16_f32, same rounding), one instruction for two values instead of half a dozen each
__host__ __device__ inline uint16_t float_to_bf16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
#else
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  uint32_t u = c.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
#endif
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int kPerChunk = 4;  // elements in one 16-byte chunk
  __device__ static inline float load(const float* p) { return *p; }
  __device__ static inline void store(float* p, float v) { *p = v; }
};
template <>
struct Elem<bf16> {
  static constexpr int kPerChunk = 8;
  __device__ static inline float load(const bf16* p) { return bf16_bits_to_float(p->v); }
  __device__ static inline void store(bf16* p, float v) { p->v = float_to_bf16_bits(v); }
};

// A 16-byte chunk as it travels global -> register -> LDS -> MFMA operand.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

union Chunk {
  uint4 u;
  uint32_t w[4];
  float f[4];
  bf16x8_t h;
};

__device__ inline Chunk zero_chunk() {
  Chunk c;
  c.u = make_uint4(0u, 0u, 0u, 0u);
  return c;
}

// unpack a chunk into fp32 lanes (E = 4 or 8)
template <typename T>
__device__ inline void chunk_to_float(const Chunk& c, float* out);
template <>
__device__ inline void chunk_to_float<float>(const Chunk& c, float* out) {
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = c.f[i];
}
template <>
__device__ inline void chunk_to_float<bf16>(const Chunk& c, float* out) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = __uint_as_float(c.w[i] << 16);
    out[2 * i + 1] = __uint_as_float(c.w[i] & 0xffff0000u);
  }
}
template <typename T>
__device__ inline Chunk float_to_chunk(const float* in);
template <>
__device__ inline Chunk float_to_chunk<float>(const float* in) {
  Chunk c;
#pragma unroll
  for (int i = 0; i < 4; ++i) c.f[i] = in[i];
  return c;
}
template <>
__device__ inline Chunk float_to_chunk<bf16>(const float* in) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  Chunk c;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f32x2_t v = {in[2 * i], in[2 * i + 1]};
    c.w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
  return c;
}

// ---------------------------------------------------------------------------
// division by a run-time constant without the integer divider
// valid for dividends in [0, 2^31)
// ---------------------------------------------------------------------------
struct FastDiv {
  uint32_t mul;
  uint32_t shr;
  uint32_t d;
  __host__ __device__ FastDiv() : mul(0), shr(0), d(1) {}
  __host__ explicit FastDiv(uint32_t denom) : mul(0), shr(0), d(denom) {
    if (denom > 1) {
      uint32_t lg = 0;
      while ((1u << lg) < denom) ++lg;  // ceil(log2(denom))
      // p = 31 + ceil(log2(d)); m = ceil(2^p / d); fits 32 bits for d >= 2
      unsigned p = 31 + lg;  // <= 62, so 2^p fits 64 bits
      uint64_t m = ((1ull << p) + denom - 1) / denom;
      mul = static_cast<uint32_t>(m);
      shr = p - 32;
    }
  }
  __device__ inline uint32_t div(uint32_t n) const { return d == 1 ? n : (__umulhi(n, mul) >> shr); }
  __device__ inline void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
    q = div(n);
    r = n - q * d;
  }
};

typedef unsigned int stream_u4 __attribute__((ext_vector_type(4)));
// 16 bytes of a tensor that is read once per pass: the caches are not asked to keep the line
__device__ inline uint4 load_streaming_u4(const void* base, int64_t i) {
  const stream_u4 v = __builtin_nontemporal_load(static_cast<const stream_u4*>(base) + i);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// 16-byte fp32 accesses that do not ask the caches to keep the line: optimizer state and master weights are touched
// once per step and are larger than every cache
typedef float stream_f4 __attribute__((ext_vector_type(4)));
__device__ inline float4 load_streaming_f4(const float* p) {
  const stream_f4 v = __builtin_nontemporal_load(reinterpret_cast<const stream_f4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ inline void store_streaming_f4(float* p, const float4& v) {
  stream_f4 s;
  s.x = v.x;
  s.y = v.y;
  s.z = v.z;
  s.w = v.w;
  __builtin_nontemporal_store(s, reinterpret_cast<stream_f4*>(p));
}

// ---------------------------------------------------------------------------
// wavefront reductions (64 lanes)
// ---------------------------------------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// ---------------------------------------------------------------------------
// exact accumulators for per-channel sums that many workgroups contribute to
// ---------------------------------------------------------------------------
// A sum over workgroups by floating-point atomics depends on the order the workgroups finish in; a sum of
// integers does not.  An accumulator is a pair of 64-bit integers: a contribution v (fp32) is split exactly
// into hi = trunc(v * 2^24) (units of 2^-24) and lo = round((v - hi * 2^-24) * 2^66) (units of 2^-66),
// each added with an integer atomic that returns nothing (no wave waits for it).  Only what lies below
// 2^-66 (1.4e-20) of a contribution is dropped, |v| < 2^38 and up to 2^20 contributions fit; the total
// hi * 2^-24 + lo * 2^-66 is the same whatever order the additions happened in, so the kernels that read it
// are bit-identical from run to run.
//
// Layout of a set of accumulators for C channels and two sums per channel: copies x [4][C] 64-bit words -- the
// planes hi(sum 0), lo(sum 0), hi(sum 1), lo(sum 1), so that the 64 lanes of one atomic instruction touch 512
// contiguous bytes.  A device-scope add costs about 20 ns per earlier add to the SAME address that is still in
// flight (measured: 1568 workgroups adding to one word take 20-35 us), so contributors are spread over `copies`
// (a power of two) by their row-tile number and the reader adds the copies up -- integers again, any order.
constexpr int kAccPlanes = 4;
__device__ inline void acc_add2(long long* acc, int C, int copies, int contributor, int c, float v0, float v1) {
  long long* base = acc + static_cast<int64_t>(contributor & (copies - 1)) * kAccPlanes * C + c;
  const float v[2] = {v0, v1};
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const double d = static_cast<double>(v[j]);
    const long long hi = static_cast<long long>(d * 16777216.0);
    const double rest = d - static_cast<double>(hi) * (1.0 / 16777216.0);
    const long long lo = __double2ll_rn(rest * 73786976294838206464.0);   // 2^66
    atomicAdd(reinterpret_cast<unsigned long long*>(base + (2 * j) * C), static_cast<unsigned long long>(hi));
    atomicAdd(reinterpret_cast<unsigned long long*>(base + (2 * j + 1) * C), static_cast<unsigned long long>(lo));
  }
}
// read by a LATER launch than the ones that added (device-scope loads: they do not trust a cached copy)
__device__ inline void acc_totals(const long long* acc, int C, int copies, int c, double* t0, double* t1) {
  long long w[kAccPlanes] = {0, 0, 0, 0};
  for (int k = 0; k < copies; ++k) {
#pragma unroll
    for (int j = 0; j < kAccPlanes; ++j)
      w[j] += __hip_atomic_load(acc + (static_cast<int64_t>(k) * kAccPlanes + j) * C + c, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
  }
  *t0 = static_cast<double>(w[0]) * (1.0 / 16777216.0) + static_cast<double>(w[1]) * (1.0 / 73786976294838206464.0);
  *t1 = static_cast<double>(w[2]) * (1.0 / 16777216.0) + static_cast<double>(w[3]) * (1.0 / 73786976294838206464.0);
}

// Workgroups are dealt round-robin to the 8 XCDs (each with a private L2).
// Remap the hardware workgroup id so that CONSECUTIVE logical ids land on the
// same XCD: neighbouring tiles then share operand rows through one L2.
__device__ inline uint32_t xcd_remap(uint32_t wg, uint32_t nwg) {
  constexpr uint32_t kXcd = 8;
  uint32_t xcd = wg % kXcd;
  uint32_t local = wg / kXcd;
  uint32_t q = nwg / kXcd, rem = nwg % kXcd;
  uint32_t start = xcd * q + (xcd < rem ? xcd : rem);
  return start + local;
}

// ---------------------------------------------------------------------------
// host side: launch sink
// ---------------------------------------------------------------------------

// Every kernel in this library takes exactly ONE trivially copyable argument
// struct by value, so a launch is (function, grid, block, bytes-of-args) and
// can be queued, recorded and replayed without knowing the kernel.
struct LaunchRecord {
  const void* fn;
  dim3 grid;
  dim3 block;
  uint32_t arg_bytes;
  // annotation for the built-in profiler: a static name and the ALGORITHMIC work of
  // this launch (flops for MFMA-bound kernels, bytes for HBM-bound ones)
  const char* name;
  double work;
  int work_is_bytes;
  // for a launch annotated with flops: its algorithmic bytes as well (0 = not given), so that a reader can
  // tell which of the two roofs binds it
  double bytes;
  // A recorded program is a valid serial order of launches.  `lane` 1 marks launches that may
  // run beside the lane-0 ones on a second stream; `op` says how the lanes meet:
  //   kOpLaunch       plain launch on its lane
  //   kOpLaunchAfter  lane-1 launch that must see everything lane 0 was given before it
  //   kOpJoin         no kernel: lane 0 waits for everything lane 1 was given so far
  //   kOpJoinBehind   no kernel: lane 0 waits for what lane 1 had been given at the PREVIOUS point of this kind
  //                   (nothing at the first one), and lane 1's work up to here is what the next one waits for
  int lane;
  int op;
  alignas(16) unsigned char args[448];
};
enum LaunchOp : int { kOpLaunch = 0, kOpLaunchAfter = 1, kOpJoin = 2, kOpJoinBehind = 3 };

// The reduction of the partial results a split weight gradient left: out (+)= sum over the splits of partial, in the
// order of the splits; optionally a second, short vector (the bias gradient) by the workgroups from first_blocks on.
struct ReduceArgs {
  const float* partial;
  float* out;
  int64_t n;
  int splits;
  int accumulate;
  const float* partial2;
  float* out2;
  int n2;
  unsigned first_blocks;
};

class Context;  // defined in context.h

int submit(Context* ctx, const void* fn, dim3 grid, dim3 block, const void* args, size_t arg_bytes,
           const char* name, double work, int work_is_bytes, double bytes = 0.0);

// name must have static storage duration
template <typename Args>
inline int launch(Context* ctx, void (*kernel)(Args), dim3 grid, dim3 block, const Args& args,
                  const char* name = "kernel", double work = 0.0, int work_is_bytes = 1, double bytes = 0.0) {
  static_assert(sizeof(Args) <= sizeof(LaunchRecord::args), "kernel argument struct too large");
  static_assert(std::is_trivially_copyable<Args>::value, "kernel arguments must be POD");
  return submit(ctx, reinterpret_cast<const void*>(kernel), grid, block, &args, sizeof(Args), name, work,
                work_is_bytes, bytes);
}

void set_error(const std::string& msg);

#define TCH_CHECK_ARG(cond, msg)                       \
  do {                                                 \
    if (!(cond)) {                                     \
      ::tch::set_error(std::string("invalid argument: ") + (msg)); \
      return -22;                                      \
    }                                                  \
  } while (0)

}  // namespace tch
