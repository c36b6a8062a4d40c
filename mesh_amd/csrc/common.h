// Shared helpers for the MoE HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/mesh_moe.h"

namespace mesh_moe {

// Per-thread error text returned by mesh_moe_last_error().
void set_error(const char* fmt, ...);

// Batched C[e] = A[e] . B[e]^T (ffn.hip): A [E,R,K], B [E,N,K] of `dtype`
// (MESH_MOE_F32 / MESH_MOE_BF16), C [E,R,N] of `dtype`, or float32 when
// out_f32.  Float32 accumulation on the matrix cores for bf16.
int batched_gemm_nt(const void* A, const void* B, void* C, int E, int R, int N,
                    int K, int dtype, bool out_f32, hipStream_t st);

// Fused self-attention (attention.hip): q, k, v, out [B,L,H*D] bf16.
bool flash_attention_supported(int L, int H, int D, int dtype, const void* q,
                               const void* k, const void* v, const void* out);
// With rel_values [H, num_buckets] bf16 and rel_bucket [2L-1] (null: none) the
// relative attention bias is added to the logits; the backward pass then
// writes its gradient to dvalues [H, num_buckets] bf16.  lse [B*H, L] float32
// (null: not wanted): the logarithm of the softmax denominators, which the
// backward pass takes back as lse_saved together with the outputs (out_saved)
// in place of recomputing them.
size_t flash_attention_workspace_bytes(int B, int L, int H, int D,
                                       bool relative_bias);
int flash_attention(const void* q, const void* k, const void* v, void* out,
                    int B, int L, int H, int D, int causal,
                    const int32_t* sequence_id, const void* rel_values,
                    const int32_t* rel_bucket, int num_buckets, float* lse,
                    void* workspace, hipStream_t st);
size_t flash_attention_backward_workspace_bytes(int B, int L, int H,
                                                bool relative_bias);
int flash_attention_backward(const void* q, const void* k, const void* v,
                             const void* dout, void* dq, void* dk, void* dv,
                             int B, int L, int H, int D, int causal,
                             const int32_t* sequence_id, const void* rel_values,
                             const int32_t* rel_bucket, int num_buckets,
                             void* dvalues, const void* out_saved,
                             const float* lse_saved, void* workspace,
                             hipStream_t st);

#define MOE_REQUIRE(cond, code, ...)      \
  do {                                    \
    if (!(cond)) {                        \
      mesh_moe::set_error(__VA_ARGS__);   \
      return (code);                      \
    }                                     \
  } while (0)

#define MOE_CHECK_LAUNCH(what)                                         \
  do {                                                                 \
    hipError_t e__ = hipGetLastError();                                \
    if (e__ != hipSuccess) {                                           \
      mesh_moe::set_error("%s: %s", (what), hipGetErrorString(e__));   \
      return MESH_MOE_E_HIP;                                           \
    }                                                                  \
  } while (0)

// Raises a kernel's dynamic-LDS limit when `bytes` exceeds the default.
#define MOE_ALLOW_LDS(kernel, bytes)                                        \
  do {                                                                      \
    if ((bytes) > 160 * 1024) {                                             \
      mesh_moe::set_error("needs %zu bytes of LDS (limit 163840)",          \
                          (size_t)(bytes));                                 \
      return MESH_MOE_E_UNSUPPORTED;                                        \
    }                                                                       \
    if ((bytes) > 32 * 1024) {                                              \
      hipError_t e__ = hipFuncSetAttribute(                                 \
          (const void*)(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,\
          (int)(bytes));                                                    \
      if (e__ != hipSuccess) {                                              \
        mesh_moe::set_error("hipFuncSetAttribute: %s",                      \
                            hipGetErrorString(e__));                        \
        return MESH_MOE_E_HIP;                                              \
      }                                                                     \
    }                                                                       \
  } while (0)

static inline bool valid_dtype(int d) {
  return d == MESH_MOE_F32 || d == MESH_MOE_BF16;
}
static inline size_t dtype_size(int d) { return d == MESH_MOE_BF16 ? 2 : 4; }

// ---- bfloat16 as raw bits -------------------------------------------------
typedef uint16_t bf16_t;

// host side: a finite float32 rounded to the nearest bfloat16 (ties to even)
static inline float round_bf16_host(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round-to-nearest-even, NaN kept quiet: gfx950's own conversion instruction
// (v_cvt_pk_bf16_f32), one issue slot instead of a compare-and-select sequence
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, (__bf16)f);
}

// two values in one instruction, `lo` in bits 15:0
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// value of `f` after a cast to the activation dtype and back
// Compacted expert rows (expert e's occupied slots, groups in order, at the
// front of its row range; row_offsets[e][g] = occupied slots of the groups
// before g): the number of occupied rows of expert e.
__device__ __forceinline__ int compact_rows_used(const int32_t* fill,
                                                 const int32_t* row_offsets,
                                                 int e, int G, int E) {
  return row_offsets[(int64_t)e * G + G - 1] + fill[(int64_t)(G - 1) * E + e];
}
// Row used + i if it lies between the occupied rows and the next multiple of
// 256 (the rows of the last occupied 256-row tile that hold no slot), else -1.
__device__ __forceinline__ int64_t compact_tail_row(int used, int i,
                                                    int64_t rows) {
  const int u = used & 255;
  const int64_t row = (int64_t)used + i;
  return (u == 0 || i >= 256 - u || row >= rows) ? -1 : row;
}

template <typename T>
__device__ __forceinline__ float round_to(float f);
template <>
__device__ __forceinline__ float round_to<float>(float f) { return f; }
template <>
__device__ __forceinline__ float round_to<bf16_t>(float f) {
  return bf16_to_f32(f32_to_bf16(f));
}

template <typename T>
__device__ __forceinline__ float load_f32(const T* p);
template <>
__device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) {
  return bf16_to_f32(*p);
}

template <typename T>
__device__ __forceinline__ void store_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_f32<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, float v) {
  *p = f32_to_bf16(v);
}

// 16-byte store that does not allocate in the L2 on its way out.  The rows
// written here are not read again by the same kernel; with ordinary stores
// the write-back L2 fetched the lines it was about to overwrite and wrote
// some of them back more than once (measured on the dispatch kernel: 1.68 GB
// written and 1.04 GB read for 1.07 GB / 0.54 GB of named traffic; with these
// stores 1.14 GB / 0.54 GB, and 0.34 ms instead of 0.43 ms).
typedef uint32_t u32x4_nt_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_streaming(uint4* p, const uint4& v) {
  __builtin_nontemporal_store(*reinterpret_cast<const u32x4_nt_t*>(&v),
                              reinterpret_cast<u32x4_nt_t*>(p));
}
// 16-byte load of data this kernel reads once (the same hint on the way in;
// the combine kernel runs 13 % faster with it).
__device__ __forceinline__ uint4 load_streaming(const uint4* p) {
  const u32x4_nt_t v =
      __builtin_nontemporal_load(reinterpret_cast<const u32x4_nt_t*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

// 16 bytes of activations <-> float32 registers
template <typename T>
struct Vec16B {
  static constexpr int N = 16 / sizeof(T);
};

__device__ __forceinline__ void unpack16(const uint4& v, float (&f)[4], float) {
  f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
  f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}
__device__ __forceinline__ void unpack16(const uint4& v, float (&f)[8], bf16_t) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}
__device__ __forceinline__ uint4 pack16(const float (&f)[4], float) {
  return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]),
                    __float_as_uint(f[2]), __float_as_uint(f[3]));
}
__device__ __forceinline__ uint4 pack16(const float (&f)[8], bf16_t) {
  uint4 r;
  r.x = f32x2_to_bf16x2(f[0], f[1]);
  r.y = f32x2_to_bf16x2(f[2], f[3]);
  r.z = f32x2_to_bf16x2(f[4], f[5]);
  r.w = f32x2_to_bf16x2(f[6], f[7]);
  return r;
}

template <typename T>
struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
};

__device__ __forceinline__ float apply_activation(float v, int act) {
  switch (act) {
    case MESH_MOE_ACT_RELU:
      return v > 0.f ? v : 0.f;
    case MESH_MOE_ACT_GELU: {
      float c = 0.5f * (1.0f + tanhf(0.7978845608028654f *
                                     (v + 0.044715f * v * v * v)));
      return v * c;
    }
    case MESH_MOE_ACT_SIGMOID:
      return 1.0f / (1.0f + expf(-v));
    case MESH_MOE_ACT_TANH:
      return tanhf(v);
    case MESH_MOE_ACT_SWISH:
      return v / (1.0f + expf(-v));
    default:
      return v;
  }
}

}  // namespace mesh_moe
