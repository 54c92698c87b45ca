// MFMA operand fragments for the fused attention kernels (bf16, 32x32x16 MFMA on gfx950), read from LDS tiles
// stored [row][column] with ROWB bytes per row.
//
// The kernels orient every product so that one side's row is the accumulator's lane (lane % 32) and the other
// side's rows are its registers: register r of lane half h = lane / 32 is row 8 (r / 4) + 4 h + r % 4.  A block
// of 8 registers 8s .. 8s+7 is then the 16 rows from 16 s in the order {8t + 4h + i}, a permutation of the 16
// reduction indices of one MFMA step; frag_cols reads the other operand of that step in the same order.
#pragma once

#include "kernels.h"

namespace tch {

typedef short attn_short4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) attn_short4_t* attn_lds_short4_ptr;
typedef __bf16 attn_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float attn_f32x2_t __attribute__((ext_vector_type(2)));

__device__ inline uint32_t pack_bf16(float a, float b) {
  attn_f32x2_t v = {a, b};
  attn_bf16x2_t r = __builtin_convertvector(v, attn_bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}

// operand fragment whose MFMA rows are tile rows row0 .. row0+31 and whose reduction index runs along the row:
// lane holds the 8 consecutive columns 16 ks + 8 (lane / 32) of row row0 + lane % 32
template <int ROWB>
__device__ inline Chunk frag_rows(const unsigned char* lds, int row0, int ks, int lane) {
  Chunk c;
  c.u = *reinterpret_cast<const uint4*>(lds + (row0 + (lane & 31)) * ROWB + (ks * 16 + 8 * (lane >> 5)) * 2);
  return c;
}

// operand fragment whose MFMA rows are the columns 32 ct .. 32 ct + 31 of the tile and whose reduction index
// runs over the 16 tile rows from row0 in the accumulator's order: element 4t + i of lane half h is row
// row0 + 8t + 4h + i (transposing LDS reads: a 16-lane group fetches a 4 x 16 patch and each lane keeps a column)
template <int ROWB>
__device__ inline Chunk frag_cols(const unsigned char* lds, int row0, int ct, int lane) {
  const int grp = lane >> 4, q16 = lane & 15;
  Chunk c;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int row = row0 + 8 * t + 4 * (grp >> 1) + (q16 >> 2);
    const int col = 32 * ct + 16 * (grp & 1) + 4 * (q16 & 3);
    union {
      attn_short4_t s;
      uint32_t w[2];
    } v;
    v.s = __builtin_amdgcn_ds_read_tr16_b64_v4i16((attn_lds_short4_ptr)(lds + row * ROWB + col * 2));
    c.w[2 * t] = v.w[0];
    c.w[2 * t + 1] = v.w[1];
  }
  return c;
}

// registers 8s .. 8s+7 of an accumulator as the second operand of the next product
__device__ inline Chunk pack_slab(const float* p) {
  Chunk c;
#pragma unroll
  for (int i = 0; i < 4; ++i) c.w[i] = pack_bf16(p[2 * i], p[2 * i + 1]);
  return c;
}

__device__ inline void zero_acc(f32x16_t& a) {
#pragma unroll
  for (int e = 0; e < 16; ++e) a[e] = 0.f;
}

__device__ inline f32x16_t mma16(const Chunk& first, const Chunk& second, f32x16_t acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(first.h, second.h, acc, 0, 0, 0);
}

}  // namespace tch
