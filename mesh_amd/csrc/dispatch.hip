// Dispatch (token rows -> expert slots), combine (expert slots -> token rows)
// and expert-weight packing for gfx950.  All three are HBM-bound row movers:
// one 64-lane wavefront moves one row with 16-byte accesses.
//
// Dispatch replaces the one-hot einsum at mesh_tensorflow/transformer/moe.py:
// 443-447, combine the einsum at moe.py:509-510; both consume the per-token
// routing record instead of the dense [G,S,E,C] tensors of moe.py:1499-1511.
#include "common.h"

namespace mesh_moe {

constexpr int ROWS_PER_BLOCK = 4;  // one wavefront per row, 256 threads

// ---------------------------------------------------------------------------
// dispatch
// jobs [0, T): token t copies its row to the slots of its kept choices (a kept
//   choice whose activation-dtype gate is exactly 0 gets a zero row: the
//   reference's dispatch tensor is bool(combine), moe.py:1510-1511);
// jobs [T, T + G*E): (g, e) zero-fills the slots fill[g,e] .. C-1.
// With row_offsets (compacted rows: expert e's occupied slots of group g start
// at row row_offsets[e][g] of its row range, as mesh_moe_compact_expert_ffn
// lays them out) the zero jobs are [T, T + 256 E) instead: job (e, i) clears
// row used(e) + i while that is below the next multiple of 256.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dispatch_kernel(
    const T* __restrict__ x, const int32_t* __restrict__ idx,
    const int32_t* __restrict__ pos, const float* __restrict__ gate,
    const uint8_t* __restrict__ kept, const int32_t* __restrict__ fill,
    T* __restrict__ expert_in, float* __restrict__ slot_gate, int G, int S,
    int E, int C, int M, int64_t T_tokens, bool vec,
    const int32_t* __restrict__ row_offsets) {
  const int lane = threadIdx.x & 63;
  const int64_t job = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  const int64_t njobs =
      T_tokens + (row_offsets != nullptr ? (int64_t)E * 256 : (int64_t)G * E);
  if (job >= njobs) return;
  if (job < T_tokens) {
    const int64_t t = job;
    const int g = (int)(t / S);
    const T* src = x + t * M;
    // The token's record in one round trip (both choices of every array at
    // once, kept or not), and -- vec path -- the first batch of the row's loads
    // issued before the record is looked at: the row's address does not
    // depend on it, and a token with no kept choice is rare.
    constexpr int VN = Vec16<T>::N;
    constexpr int UN = 8;    // 16-byte loads in flight per lane before any store
    const int nv = M / VN;
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    const uint4 z = make_uint4(0, 0, 0, 0);
    uint4 v[UN];
    if (vec) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = lane + u * 64;
        v[u] = i < nv ? load_streaming(s4 + i) : z;
      }
    }
    const uint16_t kept2 = *reinterpret_cast<const uint16_t*>(kept + t * 2);
    const int2 idx2 = *reinterpret_cast<const int2*>(idx + t * 2);
    const int2 pos2 = *reinterpret_cast<const int2*>(pos + t * 2);
    const float2 gate2 = *reinterpret_cast<const float2*>(gate + t * 2);
    T* dst[2] = {nullptr, nullptr};
    bool zero[2] = {false, false};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      if ((kept2 >> (8 * k)) & 0xff) {
        const int e = k ? idx2.y : idx2.x;
        const int c = k ? pos2.y : pos2.x;
        const float w = round_to<T>(k ? gate2.y : gate2.x);
        const int64_t slot =
            row_offsets == nullptr
                ? ((int64_t)e * G + g) * C + c
                : (int64_t)e * G * C + row_offsets[(int64_t)e * G + g] + c;
        dst[k] = expert_in + slot * M;
        zero[k] = (w == 0.0f);
        if (slot_gate != nullptr && lane == 0) slot_gate[slot] = w;
      }
    }
    if (dst[0] == nullptr && dst[1] == nullptr) return;
    if (vec) {
      uint4* d0 = reinterpret_cast<uint4*>(dst[0]);
      uint4* d1 = reinterpret_cast<uint4*>(dst[1]);
      const bool has0 = d0 != nullptr, has1 = d1 != nullptr;
      for (int base = lane; base < nv; base += 64 * UN) {
        if (base != lane) {
#pragma unroll
          for (int u = 0; u < UN; ++u) {
            const int i = base + u * 64;
            v[u] = i < nv ? load_streaming(s4 + i) : z;
          }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int i = base + u * 64;
          if (i < nv) {
            if (has0) store_streaming(d0 + i, zero[0] ? z : v[u]);
            if (has1) store_streaming(d1 + i, zero[1] ? z : v[u]);
          }
        }
      }
    } else {
      for (int i = lane; i < M; i += 64) {
        T v = src[i];
        if (dst[0]) dst[0][i] = zero[0] ? (T)0 : v;
        if (dst[1]) dst[1][i] = zero[1] ? (T)0 : v;
      }
    }
  } else if (row_offsets != nullptr) {
    const int64_t j = job - T_tokens;
    const int e = (int)(j >> 8);
    const int64_t rows = (int64_t)G * C;
    const int used = compact_rows_used(fill, row_offsets, e, G, E);
    const int64_t row = compact_tail_row(used, (int)(j & 255), rows);
    if (row < 0) return;
    T* d = expert_in + ((int64_t)e * rows + row) * M;
    if (vec) {
      constexpr int VN = Vec16<T>::N;
      uint4* d4 = reinterpret_cast<uint4*>(d);
      const uint4 z = make_uint4(0, 0, 0, 0);
      for (int i = lane; i < M / VN; i += 64) store_streaming(d4 + i, z);
    } else {
      for (int i = lane; i < M; i += 64) d[i] = (T)0;
    }
  } else {
    const int64_t ge = job - T_tokens;
    const int g = (int)(ge / E), e = (int)(ge % E);
    const int f = fill[ge];
    for (int c = f; c < C; ++c) {
      const int64_t slot = ((int64_t)e * G + g) * C + c;
      T* d = expert_in + slot * M;
      if (slot_gate != nullptr && lane == 0) slot_gate[slot] = 0.0f;
      if (vec) {
        constexpr int VN = Vec16<T>::N;
        uint4* d4 = reinterpret_cast<uint4*>(d);
        const uint4 z = make_uint4(0, 0, 0, 0);
        for (int i = lane; i < M / VN; i += 64) store_streaming(d4 + i, z);
      } else {
        for (int i = lane; i < M; i += 64) d[i] = (T)0;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// combine: out[t] = w1 * y[slot1] + w2 * y[slot2], float32 math, one rounding.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void fma2_bf16(uint32_t a, uint32_t b, float w1,
                                          float w2, uint32_t& out) {
  float a0 = __uint_as_float(a << 16), a1 = __uint_as_float(a & 0xffff0000u);
  float b0 = __uint_as_float(b << 16), b1 = __uint_as_float(b & 0xffff0000u);
  float r0 = w1 * a0 + w2 * b0;
  float r1 = w1 * a1 + w2 * b1;
  out = f32x2_to_bf16x2(r0, r1);
}

template <typename T>
__device__ __forceinline__ uint4 combine_vec(uint4 a, uint4 b, float w1,
                                             float w2);
template <>
__device__ __forceinline__ uint4 combine_vec<float>(uint4 a, uint4 b, float w1,
                                                    float w2) {
  uint4 r;
  r.x = __float_as_uint(w1 * __uint_as_float(a.x) + w2 * __uint_as_float(b.x));
  r.y = __float_as_uint(w1 * __uint_as_float(a.y) + w2 * __uint_as_float(b.y));
  r.z = __float_as_uint(w1 * __uint_as_float(a.z) + w2 * __uint_as_float(b.z));
  r.w = __float_as_uint(w1 * __uint_as_float(a.w) + w2 * __uint_as_float(b.w));
  return r;
}
template <>
__device__ __forceinline__ uint4 combine_vec<bf16_t>(uint4 a, uint4 b, float w1,
                                                     float w2) {
  uint4 r;
  fma2_bf16(a.x, b.x, w1, w2, r.x);
  fma2_bf16(a.y, b.y, w1, w2, r.y);
  fma2_bf16(a.z, b.z, w1, w2, r.z);
  fma2_bf16(a.w, b.w, w1, w2, r.w);
  return r;
}

template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(
    const T* __restrict__ y, const int32_t* __restrict__ idx,
    const int32_t* __restrict__ pos, const float* __restrict__ gate,
    const uint8_t* __restrict__ kept, T* __restrict__ out, int G, int S, int E,
    int C, int N, int64_t T_tokens, bool vec,
    const int32_t* __restrict__ row_offsets) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (t >= T_tokens) return;
  const int g = (int)(t / S);
  const T* src[2] = {nullptr, nullptr};
  float w[2] = {0.f, 0.f};
  // the token's record in one round trip (both choices of every array at
  // once, kept or not) instead of one per array
  const uint16_t kept2 = *reinterpret_cast<const uint16_t*>(kept + t * 2);
  const int2 idx2 = *reinterpret_cast<const int2*>(idx + t * 2);
  const int2 pos2 = *reinterpret_cast<const int2*>(pos + t * 2);
  const float2 gate2 = *reinterpret_cast<const float2*>(gate + t * 2);
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    if ((kept2 >> (8 * k)) & 0xff) {
      const float wk = round_to<T>(k ? gate2.y : gate2.x);
      if (wk != 0.0f) {
        const int64_t e = k ? idx2.y : idx2.x;
        const int p = k ? pos2.y : pos2.x;
        // row of the slot: [e][g][c], or with compacted rows the expert's
        // occupied slots of earlier groups first (row_offsets[e][g])
        const int64_t slot = row_offsets == nullptr
                                 ? (e * G + g) * C + p
                                 : e * G * C + row_offsets[e * G + g] + p;
        src[k] = y + slot * N;
        w[k] = wk;
      }
    }
  }
  T* dst = out + t * N;
  if (vec) {
    constexpr int VN = Vec16<T>::N;
    const int nv = N / VN;
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    const uint4* a4 = reinterpret_cast<const uint4*>(src[0]);
    const uint4* b4 = reinterpret_cast<const uint4*>(src[1]);
    const uint4 z = make_uint4(0, 0, 0, 0);
    // all loads of a batch (a whole row of 4096 bf16 from each source) are
    // issued before the first use
    constexpr int UN = 8;
    const bool has_a = a4 != nullptr, has_b = b4 != nullptr;
    for (int base = lane; base < nv; base += 64 * UN) {
      uint4 a[UN], b[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        a[u] = (has_a && i < nv) ? load_streaming(a4 + i) : z;
        b[u] = (has_b && i < nv) ? load_streaming(b4 + i) : z;
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        if (i < nv)
          store_streaming(d4 + i, combine_vec<T>(a[u], b[u], w[0], w[1]));
      }
    }
  } else {
    for (int i = lane; i < N; i += 64) {
      float a = src[0] ? load_f32<T>(src[0] + i) : 0.f;
      float b = src[1] ? load_f32<T>(src[1] + i) : 0.f;
      store_f32<T>(dst + i, w[0] * a + w[1] * b);
    }
  }
}

// ---------------------------------------------------------------------------
// pack_weights: dst[e][n][k] = (DT) src[e][k][n]   (64 x 64 tiles through LDS)
// ---------------------------------------------------------------------------
template <typename ST, typename DT>
__global__ __launch_bounds__(256) void pack_weights_kernel(
    const ST* __restrict__ src, DT* __restrict__ dst, int K, int N) {
  __shared__ float tile[64][65];
  const int e = blockIdx.z;
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const ST* s = src + (int64_t)e * K * N;
  DT* d = dst + (int64_t)e * K * N;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    int k = k0 + r, n = n0 + tx;
    tile[r][tx] = (k < K && n < N) ? load_f32<ST>(s + (int64_t)k * N + n) : 0.f;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    int n = n0 + r, k = k0 + tx;
    if (n < N && k < K) store_f32<DT>(d + (int64_t)n * K + k, tile[tx][r]);
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace mesh_moe

using namespace mesh_moe;

static int run_dispatch(const void* x, const int32_t* idx, const int32_t* pos,
                        const float* gate, const uint8_t* kept,
                        const int32_t* fill, const int32_t* row_offsets,
                        void* expert_in, float* slot_gate, int G, int S, int E,
                        int C, int M, int dtype, void* stream);

extern "C" int mesh_moe_dispatch(const void* x, const int32_t* idx,
                                 const int32_t* pos, const float* gate,
                                 const uint8_t* kept, const int32_t* fill,
                                 void* expert_in, float* slot_gate, int G,
                                 int S, int E, int C, int M, int dtype,
                                 void* stream) {
  return run_dispatch(x, idx, pos, gate, kept, fill, nullptr, expert_in,
                      slot_gate, G, S, E, C, M, dtype, stream);
}

extern "C" int mesh_moe_dispatch_compact(const void* x, const int32_t* idx,
                                         const int32_t* pos, const float* gate,
                                         const uint8_t* kept,
                                         const int32_t* fill,
                                         const int32_t* row_offsets,
                                         void* expert_in, int G, int S, int E,
                                         int C, int M, int dtype,
                                         void* stream) {
  MOE_REQUIRE(row_offsets, MESH_MOE_E_ARG, "dispatch_compact: null pointer");
  return run_dispatch(x, idx, pos, gate, kept, fill, row_offsets, expert_in,
                      nullptr, G, S, E, C, M, dtype, stream);
}

static int run_dispatch(const void* x, const int32_t* idx, const int32_t* pos,
                        const float* gate, const uint8_t* kept,
                        const int32_t* fill, const int32_t* row_offsets,
                        void* expert_in, float* slot_gate, int G, int S, int E,
                        int C, int M, int dtype, void* stream) {
  MOE_REQUIRE(x && idx && pos && gate && kept && fill && expert_in,
              MESH_MOE_E_ARG, "dispatch: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "dispatch: bad dtype %d",
              dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1, MESH_MOE_E_ARG,
              "dispatch: bad sizes G=%d S=%d E=%d C=%d M=%d", G, S, E, C, M);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t njobs =
      T_tokens + (row_offsets != nullptr ? (int64_t)E * 256 : (int64_t)G * E);
  const int64_t nblocks = (njobs + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "dispatch: too many rows (%lld)", (long long)njobs);
  const size_t es = dtype_size(dtype);
  const bool vec = ((size_t)M * es) % 16 == 0 && aligned16(x) &&
                   aligned16(expert_in);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32) {
    dispatch_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)x, idx, pos, gate, kept, fill, (float*)expert_in,
        slot_gate, G, S, E, C, M, T_tokens, vec, row_offsets);
  } else {
    dispatch_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)x, idx, pos, gate, kept, fill, (bf16_t*)expert_in,
        slot_gate, G, S, E, C, M, T_tokens, vec, row_offsets);
  }
  MOE_CHECK_LAUNCH("dispatch");
  return 0;
}

static int run_combine(const void* y, const int32_t* idx, const int32_t* pos,
                       const float* gate, const uint8_t* kept,
                       const int32_t* row_offsets, void* out, int G, int S,
                       int E, int C, int N, int dtype, void* stream);

extern "C" int mesh_moe_combine(const void* y, const int32_t* idx,
                                const int32_t* pos, const float* gate,
                                const uint8_t* kept, void* out, int G, int S,
                                int E, int C, int N, int dtype, void* stream) {
  return run_combine(y, idx, pos, gate, kept, nullptr, out, G, S, E, C, N,
                     dtype, stream);
}

extern "C" int mesh_moe_combine_compact(const void* y, const int32_t* idx,
                                        const int32_t* pos, const float* gate,
                                        const uint8_t* kept,
                                        const int32_t* row_offsets, void* out,
                                        int G, int S, int E, int C, int N,
                                        int dtype, void* stream) {
  MOE_REQUIRE(row_offsets, MESH_MOE_E_ARG, "combine_compact: null pointer");
  return run_combine(y, idx, pos, gate, kept, row_offsets, out, G, S, E, C, N,
                     dtype, stream);
}

static int run_combine(const void* y, const int32_t* idx, const int32_t* pos,
                       const float* gate, const uint8_t* kept,
                       const int32_t* row_offsets, void* out, int G, int S,
                       int E, int C, int N, int dtype, void* stream) {
  MOE_REQUIRE(y && idx && pos && gate && kept && out, MESH_MOE_E_ARG,
              "combine: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "combine: bad dtype %d",
              dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && N >= 1, MESH_MOE_E_ARG,
              "combine: bad sizes G=%d S=%d E=%d C=%d N=%d", G, S, E, C, N);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t nblocks = (T_tokens + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "combine: too many rows (%lld)", (long long)T_tokens);
  const size_t es = dtype_size(dtype);
  const bool vec = ((size_t)N * es) % 16 == 0 && aligned16(y) && aligned16(out);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32) {
    combine_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)y, idx, pos, gate, kept, (float*)out, G, S, E, C, N,
        T_tokens, vec, row_offsets);
  } else {
    combine_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)y, idx, pos, gate, kept, (bf16_t*)out, G, S, E, C, N,
        T_tokens, vec, row_offsets);
  }
  MOE_CHECK_LAUNCH("combine");
  return 0;
}

extern "C" int mesh_moe_pack_weights(const void* src, void* dst, int E, int K,
                                     int N, int src_dtype, int dst_dtype,
                                     void* stream) {
  MOE_REQUIRE(src && dst, MESH_MOE_E_ARG, "pack_weights: null pointer");
  MOE_REQUIRE(valid_dtype(src_dtype) && valid_dtype(dst_dtype), MESH_MOE_E_ARG,
              "pack_weights: bad dtype %d -> %d", src_dtype, dst_dtype);
  MOE_REQUIRE(E >= 1 && K >= 1 && N >= 1, MESH_MOE_E_ARG,
              "pack_weights: bad sizes E=%d K=%d N=%d", E, K, N);
  MOE_REQUIRE(E <= 65535 && (K + 63) / 64 <= 65535, MESH_MOE_E_UNSUPPORTED,
              "pack_weights: grid too large E=%d K=%d", E, K);
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64), (unsigned)E);
  hipStream_t st = (hipStream_t)stream;
  if (src_dtype == MESH_MOE_F32 && dst_dtype == MESH_MOE_F32)
    pack_weights_kernel<float, float><<<grid, 256, 0, st>>>(
        (const float*)src, (float*)dst, K, N);
  else if (src_dtype == MESH_MOE_F32 && dst_dtype == MESH_MOE_BF16)
    pack_weights_kernel<float, bf16_t><<<grid, 256, 0, st>>>(
        (const float*)src, (bf16_t*)dst, K, N);
  else if (src_dtype == MESH_MOE_BF16 && dst_dtype == MESH_MOE_BF16)
    pack_weights_kernel<bf16_t, bf16_t><<<grid, 256, 0, st>>>(
        (const bf16_t*)src, (bf16_t*)dst, K, N);
  else
    pack_weights_kernel<bf16_t, float><<<grid, 256, 0, st>>>(
        (const bf16_t*)src, (float*)dst, K, N);
  MOE_CHECK_LAUNCH("pack_weights");
  return 0;
}
