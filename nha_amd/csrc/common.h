// Shared device/host helpers for the gfx950 NHA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>

#include "../../include/nha_hip.h"

namespace nha {

typedef uint16_t bf16_t;  // raw bf16 bit pattern

__device__ __forceinline__ float bf16_to_f32(bf16_t x) {
  return __uint_as_float(((uint32_t)x) << 16);
}
// round-to-nearest-even, NaN stays NaN: the hardware conversion of gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}

typedef unsigned int nha_u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  // 8 consecutive elements, p 16-byte aligned
  static __device__ __forceinline__ void ld8(const float* p, float* o) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
  static __device__ __forceinline__ void st8(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
  // ld8 of data that is read once (non-temporal: it does not displace reused lines in L2)
  static __device__ __forceinline__ void ld8_stream(const float* p, float* o) {
    const nha_u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const nha_u32x4*>(p));
    const nha_u32x4 b = __builtin_nontemporal_load(reinterpret_cast<const nha_u32x4*>(p + 4));
    o[0] = __uint_as_float(a[0]); o[1] = __uint_as_float(a[1]); o[2] = __uint_as_float(a[2]); o[3] = __uint_as_float(a[3]);
    o[4] = __uint_as_float(b[0]); o[5] = __uint_as_float(b[1]); o[6] = __uint_as_float(b[2]); o[7] = __uint_as_float(b[3]);
  }
};
template <> struct Elem<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  static __device__ __forceinline__ void ld8(const bf16_t* p, float* o) {
    uint4 a = *reinterpret_cast<const uint4*>(p);
    o[0] = __uint_as_float(a.x << 16); o[1] = __uint_as_float(a.x & 0xffff0000u);
    o[2] = __uint_as_float(a.y << 16); o[3] = __uint_as_float(a.y & 0xffff0000u);
    o[4] = __uint_as_float(a.z << 16); o[5] = __uint_as_float(a.z & 0xffff0000u);
    o[6] = __uint_as_float(a.w << 16); o[7] = __uint_as_float(a.w & 0xffff0000u);
  }
  static __device__ __forceinline__ void ld8_stream(const bf16_t* p, float* o) {
    const nha_u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const nha_u32x4*>(p));
    o[0] = __uint_as_float(a[0] << 16); o[1] = __uint_as_float(a[0] & 0xffff0000u);
    o[2] = __uint_as_float(a[1] << 16); o[3] = __uint_as_float(a[1] & 0xffff0000u);
    o[4] = __uint_as_float(a[2] << 16); o[5] = __uint_as_float(a[2] & 0xffff0000u);
    o[6] = __uint_as_float(a[3] << 16); o[7] = __uint_as_float(a[3] & 0xffff0000u);
  }
  static __device__ __forceinline__ void st8(bf16_t* p, const float* v) {
    typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
    bf16x8_t a;
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = (__bf16)v[e];  // pairs convert in one packed instruction
    *reinterpret_cast<bf16x8_t*>(p) = a;
  }
};

__device__ __forceinline__ float wave_xor_f(float v, int mask) { return __shfl_xor(v, mask, 64); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// reductions over a 256-thread workgroup (red: 4 floats of LDS) and a dot product of an fp32 LDS
// vector with one global row
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
__device__ __forceinline__ float dot_row(const float* q, const T* row, int K) {
  float acc = 0.f;
  int kk = 0;
  if ((K & 7) == 0 && ((reinterpret_cast<uintptr_t>(row) & 15) == 0)) {
    for (; kk < K; kk += 8) {
      float x[8];
      Elem<T>::ld8(row + kk, x);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += q[kk + e] * x[e];
    }
    return acc;
  }
  for (; kk < K; ++kk) acc += q[kk] * Elem<T>::ld(row + kk);
  return acc;
}

static inline int next_pow2_i(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

// host-side error plumbing (thread-local message)
void set_error(const char* fmt, ...);

int layer_prologue_impl(const NhaLayerPrologueArgs* a);
int layer_epilogue_impl(const NhaLayerEpilogueArgs* a);
int layer_prologue_bwd_impl(const NhaLayerPrologueBwdArgs* a);
int layer_epilogue_bwd_parts(int rows);
int layer_epilogue_bwd_impl(const NhaLayerEpilogueBwdArgs* a);
int hybrid_prologue_impl(const NhaHybridPrologueArgs* a);
int sink_window_impl(const NhaSinkWindowArgs* a);
size_t sink_window_scratch_bytes(const NhaSinkWindowArgs* a);
int zero_sink_rescale_impl(void* o, const float* lse_swa, int B, int T, int HQ, int D, int W, int M, int dtype, void* stream);
int short_conv_impl(const NhaShortConvArgs* a);
int short_conv_bwd_parts(int T_tot);
int short_conv_bwd_impl(const NhaShortConvBwdArgs* a);
int decode_step_impl(const NhaDecodeArgs* a);
int decode_advance_impl(int32_t* count, int32_t B, void* stream);
bool decode_mfma_supported(const NhaDecodeArgs* a);
int decode_mfma_impl(const NhaDecodeArgs* a);
size_t prefill_simple_scratch_bytes(const NhaPrefillArgs* a);
// phase: 0 = whole op, 1 = state pass only, 2 = output pass only (scratch filled by an earlier state pass)
int prefill_simple_impl(const NhaPrefillArgs* a, int phase);
bool prefill_mfma_supported(const NhaPrefillArgs* a);
size_t prefill_mfma_scratch_bytes(const NhaPrefillArgs* a);
int prefill_mfma_impl(const NhaPrefillArgs* a, int phase);
int prefill_mfma_export_states(const NhaPrefillArgs* a, float* gc, float* hkc, float* hkct, float* hvct, void* hkb, void* hvb,
                               void* hkl, void* hvl, int* big);
int bwd_slot_products3(const NhaPrefillBwdArgs* a, int which, const int* big, const bf16_t* ap, const bf16_t* bp, const float* ust,
                       const float* dpst, const float* gc, const float* delta, float* dus, float* pp, float* xg, float* ck,
                       float* cv, float* dsi);
int bwd_slot_inter_slabs(const NhaPrefillBwdArgs* a);
int bwd_slot_products2(const NhaPrefillBwdArgs* a, int which, const void* hkb, const float* dus, const float* pp,
                       const float* ck, const float* cv, const float* gc, float* ek, float* ev, float* dks, float* dvs, float* dsp);
int bwd_slot_products(const NhaPrefillBwdArgs* a, const void* hkb, const void* hvb, const void* hkl, const void* hvl, bf16_t* ap, bf16_t* bp, float* ust, float* dpst,
                      float* delta, const int* big, const float* gc, float* dus, float* pp, float* xg);
bool bwd_slot_products_fuses_q(const NhaPrefillBwdArgs* a);
bool prefill_bwd_supported(const NhaPrefillBwdArgs* a);
size_t prefill_bwd_scratch_bytes(const NhaPrefillBwdArgs* a);
int prefill_bwd_impl(const NhaPrefillBwdArgs* a);
bool bwd_window_mfma_supported(const NhaPrefillBwdArgs* a);
int bwd_window_mfma_dq(const NhaPrefillBwdArgs* a, const float* delta, void* ld);
// prefill_bwd_ring.hip: the window gradients with LDS-direct operands for four query heads per kv-head at
// K = V = 128; `ld` [T_tot, HQ] pairs of floats is written by the dq call and read by the dk / dv call
bool bwd_ring_supported(const NhaPrefillBwdArgs* a);
int bwd_ring_dq(const NhaPrefillBwdArgs* a, const float* delta, float2* ld);
int bwd_ring_dkv(const NhaPrefillBwdArgs* a, const float2* ld, const float* dvs);
int bwd_window_mfma_dkv(const NhaPrefillBwdArgs* a, const float* delta, const float* dvs, const void* ld);

}  // namespace nha

#define NHA_CHECK_ARG(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      nha::set_error(__VA_ARGS__);          \
      return NHA_ERR_INVALID;               \
    }                                       \
  } while (0)

#define NHA_CHECK_LAUNCH(what)                                             \
  do {                                                                     \
    hipError_t e__ = hipGetLastError();                                    \
    if (e__ != hipSuccess) {                                               \
      nha::set_error("%s: %s", what, hipGetErrorString(e__));              \
      return NHA_ERR_LAUNCH;                                               \
    }                                                                      \
  } while (0)
