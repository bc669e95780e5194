// Matrix-core helpers of libgbx_mixers.so (gfx950: 32x32x16 bf16 MFMA, transposed LDS reads).
#pragma once
#include "mixers_common.h"

namespace gbxm {

typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// C[32 x 32] += A[32 x 16] B[16 x 32]: lane l gives A[l % 32][8 (l / 32) ..+8] and B[8 (l / 32) ..+8][l % 32] and holds
// C[8 (e / 4) + 4 (l / 32) + e % 4][l % 32], e = 0..15.
__device__ __forceinline__ f32x16 mfma_bf16(const u32x4& a, const u32x4& b, const f32x16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// two fp32 -> one packed bf16 pair, round to nearest even
__device__ __forceinline__ unsigned pack2(float a, float b) {
  f32x2v v; v.x = a; v.y = b;
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2v));
}
// ds_read_b64_tr_b16: per 16-lane group a 4-row x 16-column block of 16-bit elements, delivered column-major (lane i of the group:
// column i, rows 0..3); lane 4q + p of the group supplies the address of row q, columns 4p .. 4p+3.  EXEC must be full.
__device__ __forceinline__ u32x2 lds_read_tr(const unsigned char* p) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (s16x4 __attribute__((address_space(3)))*)(__attribute__((address_space(3))) unsigned char*)p));
}

}  // namespace gbxm
