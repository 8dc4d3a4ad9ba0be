// Device-side helpers shared by the gfx950 kernels: bf16 packing, MFMA wrappers and
// LDS operand loads.  wave = 64 lanes throughout.
//
// MFMA operand layouts used here (verified on hardware against a CPU matmul):
//   v_mfma_f32_16x16x32_bf16  A: lane l holds row (l%16),  k = 8*(l/16)+j   j<8
//                             B: lane l holds col (l%16),  k = 8*(l/16)+j
//                             C: lane l holds col (l%16),  rows 4*(l/16)+r  r<4
//   v_mfma_f32_32x32x16_bf16  A: lane l holds row (l%32),  k = 8*(l/32)+j
//                             B: lane l holds col (l%32),  k = 8*(l/32)+j
//                             C: lane l holds col (l%32),  rows 8*(r/4)+4*(l/32)+(r%4)  r<16
//   ds_read_b64_tr_b16        within each group of 16 lanes, lane i supplies the address of
//                             a 4-element row R_i; lane i receives { R_{4j + i/4}[i%4] : j<4 }.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natsl {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

typedef uint16_t bf16_t;  // raw bits

#define NATSL_DEVICE __device__ __forceinline__

NATSL_DEVICE float bf16_to_f32(bf16_t b) { return __uint_as_float(((unsigned)b) << 16); }

// round-to-nearest-even through the hardware conversion (v_cvt_pk_bf16_f32)
NATSL_DEVICE unsigned pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}

NATSL_DEVICE bf16_t f32_to_bf16(float f) { return (bf16_t)(pack_bf16x2(f, 0.f) & 0xffffu); }

// 8 fp32 -> one bf16x8 operand: slots 0..3 from a, 4..7 from b
NATSL_DEVICE bf16x8 pack8(const f32x4 a, const f32x4 b) {
  u32x4 w;
  w[0] = pack_bf16x2(a[0], a[1]);
  w[1] = pack_bf16x2(a[2], a[3]);
  w[2] = pack_bf16x2(b[0], b[1]);
  w[3] = pack_bf16x2(b[2], b[3]);
  return __builtin_bit_cast(bf16x8, w);
}

NATSL_DEVICE f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
NATSL_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// 16-byte LDS / global loads of 8 bf16 as an MFMA operand
NATSL_DEVICE bf16x8 ld8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

NATSL_DEVICE bf16x8 zero8() {
  u32x4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

// Transposing LDS read: see the layout note at the top of this file.
NATSL_DEVICE s16x4 lds_tr4(const bf16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

NATSL_DEVICE bf16x8 join4(s16x4 lo, s16x4 hi) {
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

// x[lane ^ 32] combined symmetrically: both returned words together hold {own, partner}.
NATSL_DEVICE float xhalf_max(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
NATSL_DEVICE float xhalf_sum(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Per-sequence descriptor for packed (variable-length) input; one row per sequence.
struct SeqRow {
  int bos;        // first token (flat index)
  int eos;        // one past the last token
  int bos_nats;   // first selector block (flat index)
  int chunk_off;  // number of 64-token chunks in earlier sequences
  int qtile_off;  // number of softmax query tiles in earlier sequences
  int pad0, pad1, pad2;
};

}  // namespace natsl
