// Backward of the Mixture-of-Experts layer for gfx950: the token-side kernels.
//
// The reference has no backward code of its own for the layer: mtf.gradients
// (mesh_tensorflow/ops.py:5254-5291) assembles it from the gradients of the
// einsums and element-wise ops the layer is built from
// (EinsumOperation.gradient ops.py:2846-2854, TopKOperation.gradient
// ops.py:4916-4920, softmax ops.py:5493-5541).  With the one-hot
// dispatch / combine tensors of transformer/moe.py:1499-1511 replaced by the
// per-token routing record, those einsum gradients become the gathers and
// scatters below.  The expert feed-forward backward (four grouped GEMMs) lives
// next to the forward GEMM.
#include "common.h"

namespace mesh_moe {

constexpr int BW_ROWS_PER_BLOCK = 4;  // one wavefront per row, 256 threads

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---------------------------------------------------------------------------
// combine backward.  Forward: out[t] = w1 * y[slot1] + w2 * y[slot2] with
// w_k the activation-dtype gate (transformer/moe.py:509-510).  Hence
//   dy[slot_k]  = w_k * dout[t]            (rounded to the activation dtype)
//   dgate[t,k]  = <dout[t], y[slot_k]>     (float32), 0 where not kept
// Jobs [0, T): tokens; jobs [T, T + G*E): zero rows for the slots >= fill.
// With row_offsets, y and dy hold every expert's occupied slots at the front
// of its row range (slots of group g from row row_offsets[e][g]); the zero
// jobs are then [T, T + 256 E): the rows between an expert's occupied rows
// and the next multiple of 256.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void combine_backward_kernel(
    const T* __restrict__ dout, const T* __restrict__ y,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ pos,
    const float* __restrict__ gate, const uint8_t* __restrict__ kept,
    const int32_t* __restrict__ fill, T* __restrict__ dy,
    float* __restrict__ dgate, int G, int S, int E, int C, int N,
    int64_t T_tokens, bool vec, const int32_t* __restrict__ row_offsets) {
  constexpr int VN = Vec16B<T>::N;
  const int lane = threadIdx.x & 63;
  const int64_t job =
      (int64_t)blockIdx.x * BW_ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (job >= T_tokens +
                 (row_offsets != nullptr ? (int64_t)E * 256 : (int64_t)G * E))
    return;
  if (job >= T_tokens && row_offsets != nullptr) {
    const int64_t j = job - T_tokens;
    const int e = (int)(j >> 8);
    const int64_t rows = (int64_t)G * C;
    const int64_t row = compact_tail_row(
        compact_rows_used(fill, row_offsets, e, G, E), (int)(j & 255), rows);
    if (row < 0) return;
    T* d = dy + ((int64_t)e * rows + row) * N;
    if (vec) {
      uint4* d4 = reinterpret_cast<uint4*>(d);
      for (int i = lane; i < N / VN; i += 64)
        store_streaming(d4 + i, make_uint4(0, 0, 0, 0));
    } else {
      for (int i = lane; i < N; i += 64) d[i] = (T)0;
    }
    return;
  }
  if (job >= T_tokens) {
    const int64_t ge = job - T_tokens;
    const int g = (int)(ge / E), e = (int)(ge % E);
    for (int c = fill[ge]; c < C; ++c) {
      T* d = dy + (((int64_t)e * G + g) * C + c) * N;
      if (vec) {
        uint4* d4 = reinterpret_cast<uint4*>(d);
        for (int i = lane; i < N / VN; i += 64)
          store_streaming(d4 + i, make_uint4(0, 0, 0, 0));
      } else {
        for (int i = lane; i < N; i += 64) d[i] = (T)0;
      }
    }
    return;
  }
  const int64_t t = job;
  const int g = (int)(t / S);
  const T* yrow[2] = {nullptr, nullptr};
  T* drow[2] = {nullptr, nullptr};
  float w[2] = {0.f, 0.f};
  // the token's record in one round trip (both choices of every array at once)
  const uint16_t kept2 = *reinterpret_cast<const uint16_t*>(kept + t * 2);
  const int2 idx2 = *reinterpret_cast<const int2*>(idx + t * 2);
  const int2 pos2 = *reinterpret_cast<const int2*>(pos + t * 2);
  const float2 gate2 = *reinterpret_cast<const float2*>(gate + t * 2);
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    if ((kept2 >> (8 * k)) & 0xff) {
      const int64_t e = k ? idx2.y : idx2.x;
      const int64_t slot =
          (row_offsets == nullptr ? (e * G + g) * C
                                  : e * G * C + row_offsets[e * G + g]) +
          (k ? pos2.y : pos2.x);
      yrow[k] = y + slot * N;
      drow[k] = dy + slot * N;
      w[k] = round_to<T>(k ? gate2.y : gate2.x);
    }
  }
  float dot[2] = {0.f, 0.f};
  const T* drc = dout + t * N;
  if (vec) {
    const uint4* d4 = reinterpret_cast<const uint4*>(drc);
    const int nv = N / VN;
    // the loads of eight 16-byte steps (dout and both y rows: whole rows of
    // 4096 bf16) are issued before the first use (0.486 ms against 0.545 ms
    // with one step at a time, 65536 tokens of 4096 bf16)
    constexpr int UN = 8;
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int base = lane; base < nv; base += 64 * UN) {
      uint4 dr[UN], yr[2][UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        dr[u] = i < nv ? load_streaming(d4 + i) : z;
#pragma unroll
        for (int k = 0; k < 2; ++k)
          yr[k][u] = (yrow[k] != nullptr && i < nv)
                         ? load_streaming(
                               reinterpret_cast<const uint4*>(yrow[k]) + i)
                         : z;
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        if (i >= nv) continue;
        float d[VN];
        unpack16(dr[u], d, T());
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          if (yrow[k] == nullptr) continue;
          float yv[VN], o[VN];
          unpack16(yr[k][u], yv, T());
#pragma unroll
          for (int j = 0; j < VN; ++j) {
            dot[k] += d[j] * yv[j];
            o[j] = w[k] * d[j];
          }
          store_streaming(reinterpret_cast<uint4*>(drow[k]) + i, pack16(o, T()));
        }
      }
    }
  } else {
    for (int i = lane; i < N; i += 64) {
      const float d = load_f32<T>(drc + i);
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        if (yrow[k] == nullptr) continue;
        dot[k] += d * load_f32<T>(yrow[k] + i);
        store_f32<T>(drow[k] + i, w[k] * d);
      }
    }
  }
  dot[0] = wave_sum(dot[0]);
  dot[1] = wave_sum(dot[1]);
  if (lane == 0) {
    dgate[t * 2 + 0] = yrow[0] ? dot[0] : 0.f;
    dgate[t * 2 + 1] = yrow[1] ? dot[1] : 0.f;
  }
}

// ---------------------------------------------------------------------------
// dispatch backward (+ router projection backward w.r.t. the tokens).
// Forward: expert_in[slot_k] = x[t] for every dispatched choice (a kept choice
// whose activation-dtype gate is non-zero, transformer/moe.py:443-447,
// :1510-1511) and logits[t] = float(x[t]) . w_gate (moe.py:1384-1390).  Hence
//   dx[t] = sum_k dispatched_k * dexpert_in[slot_k] + dlogits[t] . w_gate^T
// float32 accumulate, one rounding.  w_gate comes K-contiguous ([E, M]), one
// per `groups_per_router` consecutive groups (the inner level of the
// hierarchical layer has a router per outer expert, moe.py:743-753).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dispatch_backward_kernel(
    const T* __restrict__ dxe, const int32_t* __restrict__ idx,
    const int32_t* __restrict__ pos, const float* __restrict__ gate,
    const uint8_t* __restrict__ kept, const float* __restrict__ dlogits,
    const T* __restrict__ wgp, T* __restrict__ dx, int G, int S, int E, int C,
    int M, int64_t T_tokens, int groups_per_router, bool vec,
    const int32_t* __restrict__ row_offsets) {
  constexpr int VN = Vec16B<T>::N;
  const int lane = threadIdx.x & 63;
  const int64_t t =
      (int64_t)blockIdx.x * BW_ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (t >= T_tokens) return;
  const int g = (int)(t / S);
  if (wgp != nullptr) wgp += (int64_t)(g / groups_per_router) * E * M;
  const T* src[2] = {nullptr, nullptr};
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    if (kept[t * 2 + k] && round_to<T>(gate[t * 2 + k]) != 0.0f) {
      const int64_t e = idx[t * 2 + k];
      const int64_t slot =
          (row_offsets == nullptr ? (e * G + g) * C
                                  : e * G * C + row_offsets[e * G + g]) +
          pos[t * 2 + k];
      src[k] = dxe + slot * M;
    }
  }
  const float* dl = dlogits ? dlogits + t * E : nullptr;
  T* dst = dx + t * M;
  if (vec) {
    for (int i = lane; i < M / VN; i += 64) {
      float acc[VN];
#pragma unroll
      for (int j = 0; j < VN; ++j) acc[j] = 0.f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        if (src[k] == nullptr) continue;
        float v[VN];
        unpack16(load_streaming(reinterpret_cast<const uint4*>(src[k]) + i), v,
                 T());
#pragma unroll
        for (int j = 0; j < VN; ++j) acc[j] += v[j];
      }
      if (dl != nullptr) {
        for (int e = 0; e < E; ++e) {
          const float d = dl[e];
          float v[VN];
          unpack16(reinterpret_cast<const uint4*>(wgp + (int64_t)e * M)[i], v,
                   T());
#pragma unroll
          for (int j = 0; j < VN; ++j) acc[j] += d * v[j];
        }
      }
      store_streaming(reinterpret_cast<uint4*>(dst) + i, pack16(acc, T()));
    }
  } else {
    for (int i = lane; i < M; i += 64) {
      float acc = 0.f;
      if (src[0]) acc += load_f32<T>(src[0] + i);
      if (src[1]) acc += load_f32<T>(src[1] + i);
      if (dl != nullptr)
        for (int e = 0; e < E; ++e)
          acc += dl[e] * load_f32<T>(wgp + (int64_t)e * M + i);
      store_f32<T>(dst + i, acc);
    }
  }
}

// The same with the router's share for FOUR tokens per wavefront: a 16-byte
// piece of a router kernel row, once loaded, serves all four (the one-token
// kernel reads the whole router kernel, E * M elements, per token, which is
// what bounds it).  The four tokens' d(logits) sit in LDS as [e][4], so one
// broadcast read per expert feeds 4 x 8 multiply-adds.  Needs 16-byte rows,
// E <= DBR_MAX_E and S % 4 == 0 (the four tokens share a group).
constexpr int DBR_TOK = 4;
constexpr int DBR_MAX_E = 128;

template <typename T>
__global__ __launch_bounds__(256) void dispatch_backward_router4_kernel(
    const T* __restrict__ dxe, const int32_t* __restrict__ idx,
    const int32_t* __restrict__ pos, const float* __restrict__ gate,
    const uint8_t* __restrict__ kept, const float* __restrict__ dlogits,
    const T* __restrict__ wgp, T* __restrict__ dx, int G, int S, int E, int C,
    int M, int64_t T_tokens, int groups_per_router,
    const int32_t* __restrict__ row_offsets) {
  constexpr int VN = Vec16B<T>::N;
  __shared__ __attribute__((aligned(16))) float dls[4][DBR_MAX_E][DBR_TOK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t0 = ((int64_t)blockIdx.x * 4 + wave) * DBR_TOK;
  if (t0 >= T_tokens) return;          // whole wavefronts leave: no barrier below
  const int g = (int)(t0 / S);
  wgp += (int64_t)(g / groups_per_router) * E * M;
  const T* src[DBR_TOK][2];
#pragma unroll
  for (int j = 0; j < DBR_TOK; ++j) {
    const int64_t t = t0 + j;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      src[j][k] = nullptr;
      if (t < T_tokens && kept[t * 2 + k] &&
          round_to<T>(gate[t * 2 + k]) != 0.0f) {
        const int64_t e = idx[t * 2 + k];
        const int64_t slot =
            (row_offsets == nullptr ? (e * G + g) * C
                                    : e * G * C + row_offsets[e * G + g]) +
            pos[t * 2 + k];
        src[j][k] = dxe + slot * M;
      }
    }
  }
  // this wavefront's d(logits) -> LDS, transposed to [e][token]
  for (int i = lane; i < E * DBR_TOK; i += 64) {
    const int j = i / E, e = i - j * E;
    dls[wave][e][j] = t0 + j < T_tokens ? dlogits[(t0 + j) * E + e] : 0.f;
  }
  // (same wavefront writes and reads: program order is enough within a wave)
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
  for (int i = lane; i < M / VN; i += 64) {
    float acc[DBR_TOK][VN];
#pragma unroll
    for (int j = 0; j < DBR_TOK; ++j) {
#pragma unroll
      for (int q = 0; q < VN; ++q) acc[j][q] = 0.f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        if (src[j][k] == nullptr) continue;
        float v[VN];
        unpack16(load_streaming(reinterpret_cast<const uint4*>(src[j][k]) + i), v,
                 T());
#pragma unroll
        for (int q = 0; q < VN; ++q) acc[j][q] += v[q];
      }
    }
    for (int e = 0; e < E; ++e) {
      float w[VN];
      unpack16(reinterpret_cast<const uint4*>(wgp + (int64_t)e * M)[i], w, T());
      const float4 d4 = *reinterpret_cast<const float4*>(&dls[wave][e][0]);
      const float d[DBR_TOK] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
      for (int j = 0; j < DBR_TOK; ++j)
#pragma unroll
        for (int q = 0; q < VN; ++q) acc[j][q] = fmaf(d[j], w[q], acc[j][q]);
    }
#pragma unroll
    for (int j = 0; j < DBR_TOK; ++j)
      if (t0 + j < T_tokens)
        store_streaming(reinterpret_cast<uint4*>(dx + (t0 + j) * M) + i,
                        pack16(acc[j], T()));
  }
}

// The same for bfloat16 with the router's share on the matrix cores
// (v_mfma_f32_32x32x16_bf16).  The share of 32 tokens x 256 columns,
// sum_e dlogits[t][e] * w_gate[m][e], is a product whose two operands both lie
// in memory with e innermost: the router kernel in its variable layout
// [M, E] and d(logits) [T, E].  The block copies its 256 kernel rows and 32
// d(logits) rows to LDS with whole-line loads (lanes reading their 8
// consecutive e straight from global memory touch 32 lines per instruction and
// ask for every line four times: 0.59 against 0.49 ms for 65536 tokens of 4096)
// and the lanes take their operands from there.  The float32 d(logits) go in as two bfloat16 terms
// (hi = bf16(d), lo = bf16(d - hi): the products are exact in the float32
// accumulator, what is dropped is below 2^-17 |d|).  The instruction leaves a
// lane with 4 consecutive columns of one token; the tile goes through LDS as
// float32 (over the kernel rows, which are no longer needed) so that the
// second phase -- half a wavefront per token row, 16 bytes per lane, the rows
// of d(expert_in) added -- reads and writes whole rows.  The rows' loads are
// issued before the first phase, whose latency they hide.  KS = E / 16.
// Needs M % 256 == 0, E % 16 == 0, E <= DBM_MAX_E, S % 32 == 0 (the 32 tokens
// share a group).
constexpr int DBM_TOK = 32, DBM_COLS = 256, DBM_MAX_E = 128;
constexpr int DBM_LD = DBM_COLS + 4;     // floats per LDS row of the share
typedef __attribute__((ext_vector_type(8))) __bf16 dbm_bf16x8_t;
typedef float dbm_f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t dbm_u32x4_t __attribute__((ext_vector_type(4)));

// LDS bytes: [kernel rows | share] then the d(logits) rows
static size_t dbm_lds_bytes(int E) {
  const size_t wbytes = (size_t)DBM_COLS * (E * 2 + 16);
  const size_t sbytes = sizeof(float) * DBM_TOK * DBM_LD;
  return (wbytes > sbytes ? wbytes : sbytes) + (size_t)DBM_TOK * (E * 4 + 16);
}

// Block barrier that waits for this wavefront's LDS accesses only.
__device__ __forceinline__ void dbm_lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// (Four token tiles per block with the kernel rows kept in registers and the
// next tile's loads in flight: 0.60 against 0.50 ms.)
// SLOT: the rows of a token are named by the token -> slot table of the
// expert-selection router (tok_slot [T, E] int16, -1 = not chosen by that
// expert; any number of rows per token) instead of the per-token record.
// COMPACT: the rows lie in the compacted order (row_offsets given).
template <int KS, bool SLOT = false, bool COMPACT = false>
__global__ __launch_bounds__(256) void dispatch_backward_mfma_kernel(
    const bf16_t* __restrict__ dxe, const int32_t* __restrict__ idx,
    const int32_t* __restrict__ pos, const float* __restrict__ gate,
    const uint8_t* __restrict__ kept, const float* __restrict__ dlogits,
    const bf16_t* __restrict__ wg, bf16_t* __restrict__ dx, int G, int S,
    int C, int M, int64_t T_tokens, int groups_per_router,
    const int32_t* __restrict__ row_offsets,
    const int16_t* __restrict__ tok_slot = nullptr) {
  constexpr int E = KS * 16;
  constexpr int WROW = E * 2 + 16, DROW = E * 4 + 16;   // padded LDS rows, bytes
  constexpr int WBYTES = DBM_COLS * WROW;
  constexpr int SBYTES = (int)sizeof(float) * DBM_TOK * DBM_LD;
  extern __shared__ __attribute__((aligned(16))) unsigned char dbm_smem[];
  unsigned char* wl = dbm_smem;
  float* share = reinterpret_cast<float*>(dbm_smem);
  unsigned char* dl = dbm_smem + (WBYTES > SBYTES ? WBYTES : SBYTES);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int64_t t0 = (int64_t)blockIdx.y * DBM_TOK;
  const int m0 = blockIdx.x * DBM_COLS;
  const int g = (int)(t0 / S);
  wg += (int64_t)(g / groups_per_router) * M * E;

  constexpr int WPR = E / 8;                  // 16-byte pieces per kernel row
  constexpr int WP = DBM_COLS * WPR / 256;    // pieces per thread (= E / 8)
  constexpr int DPR = E / 4;                  // pieces per d(logits) row
  constexpr int DP = (DBM_TOK * DPR + 255) / 256;
  constexpr int RP = DBM_TOK / 8;
  const uint4 z = make_uint4(0, 0, 0, 0);

  // Issue order (vmcnt retires in order, and nothing below waits for more
  // than it needs): the tokens' records, the kernel rows, the d(logits) rows,
  // and last the rows of d(expert_in), which stay in flight through the whole
  // matrix phase.  Every load is unconditional -- for a row that is not kept
  // slot 0 is read and dropped -- so the code up to phase 2 is one basic block
  // and the waits count exactly.  The barriers wait for LDS only
  // (__syncthreads() would wait for the rows as well).
  // Records: token rows wave * 8 + 2 j + half, both choices of every array in
  // one load each.
  uint16_t kept2[RP];
  int2 idx2[RP], pos2[RP];
  float2 gate2[RP];
  if constexpr (!SLOT) {
#pragma unroll
    for (int j = 0; j < RP; ++j) {
      int64_t t = t0 + wave * 8 + 2 * j + half;
      t = t < T_tokens ? t : T_tokens - 1;
      kept2[j] = *reinterpret_cast<const uint16_t*>(kept + t * 2);
      idx2[j] = *reinterpret_cast<const int2*>(idx + t * 2);
      pos2[j] = *reinterpret_cast<const int2*>(pos + t * 2);
      gate2[j] = *reinterpret_cast<const float2*>(gate + t * 2);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // (written as asm so that they are issued here: the compiler moves ordinary
  // loads of the kernel rows behind the rows of d(expert_in), next to their
  // use, and the wait for them then waits for everything)
  dbm_u32x4_t wv[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const uint4* src =
        reinterpret_cast<const uint4*>(wg + (int64_t)m0 * E) + tid + 256 * i;
    asm volatile("global_load_dwordx4 %0, %1, off"
                 : "=&v"(wv[i]) : "v"(src) : "memory");
  }
  float4 dv[DP];
  bool dv_used[DP];
#pragma unroll
  for (int i = 0; i < DP; ++i) {
    const int p = tid + 256 * i;
    dv_used[i] = p < DBM_TOK * DPR && t0 + p / DPR < T_tokens;
    dv[i] = reinterpret_cast<const float4*>(dlogits + t0 * E)[dv_used[i] ? p : 0];
  }
  __builtin_amdgcn_sched_barrier(0);
  // the rows this lane adds in phase 2: 8 columns from column 8 l32 of the tile
  // (bit 2 j + k of `used`: the row counts; the others are loaded from slot 0)
  uint4 v[RP][2];
  unsigned used = 0;
  if constexpr (!SLOT) {
    int64_t base[RP][2];
#pragma unroll
    for (int j = 0; j < RP; ++j)
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int64_t e = k ? idx2[j].y : idx2[j].x;
        if constexpr (COMPACT)
          base[j][k] = e * G * C + row_offsets[e * G + g];
        else
          base[j][k] = (e * G + g) * C;
      }
#pragma unroll
    for (int j = 0; j < RP; ++j) {
      const bool in_range = t0 + wave * 8 + 2 * j + half < T_tokens;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const float gk = round_to<bf16_t>(k ? gate2[j].y : gate2[j].x);
        const bool u =
            in_range & (((kept2[j] >> (8 * k)) & 0xff) != 0) & (gk != 0.0f);
        used |= (u ? 1u : 0u) << (2 * j + k);
        const int64_t slot = u ? base[j][k] + (k ? pos2[j].y : pos2[j].x) : 0;
        v[j][k] = load_streaming(
            reinterpret_cast<const uint4*>(dxe + slot * M + m0) + l32);
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- the kernel rows and the d(logits) rows: registers -> LDS -> operands
  // (the kernel rows have landed when only the 2 RP row loads issued after
  // them may still be in flight)
  if constexpr (SLOT)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * RP) : "memory");
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int p = tid + 256 * i;
    *reinterpret_cast<dbm_u32x4_t*>(wl + (p / WPR) * WROW + (p % WPR) * 16) =
        wv[i];
  }
#pragma unroll
  for (int i = 0; i < DP; ++i) {
    const int p = tid + 256 * i;
    if (p < DBM_TOK * DPR)
      *reinterpret_cast<float4*>(dl + (p / DPR) * DROW + (p % DPR) * 16) =
          dv_used[i] ? dv[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  dbm_lds_barrier();
  uint4 afrag[2][KS];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      afrag[b][ks] = *reinterpret_cast<const uint4*>(
          wl + (wave * 64 + b * 32 + l32) * WROW + ks * 32 + half * 16);
  {
    // ---- phase 1: this wavefront's 32 tokens x 64 columns of the share
    dbm_f32x16_t acc[2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 d0 = *reinterpret_cast<const float4*>(dl + l32 * DROW + ks * 64 + half * 32);
      const float4 d1 = *reinterpret_cast<const float4*>(dl + l32 * DROW + ks * 64 + half * 32 + 16);
      const float d[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
      float lo[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) lo[j] = d[j] - round_to<bf16_t>(d[j]);
      const dbm_bf16x8_t bh = __builtin_bit_cast(dbm_bf16x8_t, pack16(d, bf16_t()));
      const dbm_bf16x8_t bl = __builtin_bit_cast(dbm_bf16x8_t, pack16(lo, bf16_t()));
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const dbm_bf16x8_t a = __builtin_bit_cast(dbm_bf16x8_t, afrag[b][ks]);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bh, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bl, acc[b], 0, 0, 0);
      }
    }
    // (the share goes over the kernel rows: every wavefront has its operands
    // in registers before the first write)
    dbm_lds_barrier();
    // lane: token l32, columns 32 b + 8 q + 4 half + 0..3 of the wavefront's 64
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<float4*>(
            &share[l32 * DBM_LD + wave * 64 + b * 32 + q * 8 + half * 4]) =
            make_float4(acc[b][4 * q], acc[b][4 * q + 1], acc[b][4 * q + 2],
                        acc[b][4 * q + 3]);
    dbm_lds_barrier();

    // ---- phase 2
#pragma unroll
    for (int j = 0; j < RP; ++j) {
      const int row = wave * 8 + 2 * j + half;
      const int64_t t = t0 + row;
      if (t >= T_tokens) continue;
      const float* sh = &share[row * DBM_LD + l32 * 8];
      const float4 s0 = *reinterpret_cast<const float4*>(sh);
      const float4 s1 = *reinterpret_cast<const float4*>(sh + 4);
      // (the order of the one-token kernel: the rows first, then the share)
      float a[8], b[8], o[8];
      if constexpr (SLOT) {
        // this half-wavefront's token: lane l32 looks at experts l32, l32 + 32,
        // ..; the rows are added in expert order
#pragma unroll
        for (int q = 0; q < 8; ++q) { a[q] = 0.f; b[q] = 0.f; }
        for (int e0 = 0; e0 < E; e0 += 32) {
          const int c = e0 + l32 < E ? (int)tok_slot[t * E + e0 + l32] : -1;
          unsigned m = (unsigned)(__ballot(c >= 0) >> (32 * half));
          while (m != 0u) {
            const int el = __builtin_ctz(m);
            m &= m - 1u;
            const int64_t cc = __shfl(c, half * 32 + el, 64);
            const int64_t slot = ((int64_t)(e0 + el) * G + g) * C + cc;
            float r[8];
            unpack16(load_streaming(reinterpret_cast<const uint4*>(
                         dxe + slot * M + m0) + l32), r, bf16_t());
#pragma unroll
            for (int q = 0; q < 8; ++q) a[q] += r[q];
          }
        }
      } else {
        unpack16(v[j][0], a, bf16_t());
        unpack16(v[j][1], b, bf16_t());
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          a[q] = (used >> (2 * j)) & 1u ? a[q] : 0.f;
          b[q] = (used >> (2 * j + 1)) & 1u ? b[q] : 0.f;
        }
      }
      const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] = (a[q] + b[q]) + sv[q];
      store_streaming(reinterpret_cast<uint4*>(dx + t * M + m0) + l32,
                      pack16(o, bf16_t()));
    }
  }
}

// ---------------------------------------------------------------------------
// gating backward.
// Step 1, one block per group: how many tokens count for density_1 of each
// expert and how many tokens have importance 1.
// Step 2, one thread per token: d(logits) from d(gates) and d(loss).
// ---------------------------------------------------------------------------
struct GateBackwardParams {
  int G, S, E;
  int router;           // 0 = top-2, 1 = switch / switch_max, 2 = ntlb
  int top_k;            // ntlb: candidates per token
  int use_second_place_loss;  // top-2: the loss has the density_2 term too
  int has_importance;
  int importance_from_slot_gate;  // importance = 0.5*((w>0.5)+(w>0))
  int num_microbatches;
  int use_z_loss;
  float z_loss_coef;
  float loss_scale;     // moe_loss_coef as the activation dtype holds it
  int softmax_bf16;     // ntlb with bfloat16 activations: the forward rounded
                        // the logits and every softmax op to bfloat16
};

// The forward's softmax of one row: lse_out = log-sum-exp as the forward
// formed it; the probability of entry e is then gb_prob(row[e], neglse, bf).
// bf: every op's result rounded to bfloat16 (ntlb_softmax_row of the forward
// kernel), else plain float32.
__device__ __forceinline__ float gb_round(float v, bool bf) {
  return bf ? round_to<bf16_t>(v) : v;
}
__device__ __forceinline__ float gb_logsumexp(const float* row, int E, bool bf) {
  float m = gb_round(row[0], bf);
  for (int e = 1; e < E; ++e) m = fmaxf(m, gb_round(row[e], bf));
  const float negm = -m;
  float s = 0.f;
  for (int e = 0; e < E; ++e)
    s += gb_round(expf(gb_round(gb_round(row[e], bf) + negm, bf)), bf);
  s = gb_round(s, bf);
  return gb_round(gb_round(logf(s), bf) + m, bf);
}
__device__ __forceinline__ float gb_prob(float logit, float neglse, bool bf) {
  return gb_round(expf(gb_round(gb_round(logit, bf) + neglse, bf)), bf);
}

constexpr int GB_MAX_K = 8;

template <typename IT>
__global__ __launch_bounds__(256) void gate_count_kernel(
    GateBackwardParams p, const float* __restrict__ logits,
    const int32_t* __restrict__ idx, const IT* __restrict__ importance,
    int32_t* __restrict__ counts, float* __restrict__ n_one) {
  extern __shared__ int32_t cnt[];  // [E] + 1 + [E]
  int32_t* cnt2 = cnt + p.E + 1;    // second choices (second-place loss)
  // block (g, chunk): its share of the group's tokens, added to the group's
  // counters (zero before the launch) with integer-valued atomics
  const int g = blockIdx.x;
  const int per = (p.S + gridDim.y - 1) / gridDim.y;
  const int s_lo = blockIdx.y * per, s_hi = min(p.S, s_lo + per);
  for (int e = threadIdx.x; e <= 2 * p.E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int s = s_lo + threadIdx.x; s < s_hi; s += blockDim.x) {
    const int64_t t = (int64_t)g * p.S + s;
    bool one = true, positive = true;
    if (importance != nullptr) {
      const float imp = load_f32<IT>(importance + t);
      // from a slot weight w: 0.5*((w>0.5)+(w>0)) == 1  <=>  w > 0.5
      one = p.importance_from_slot_gate ? imp > 0.5f : imp == 1.0f;
      positive = imp > 0.0f;    // either form: 0.5*((w>0.5)+(w>0)) > 0 <=> w > 0
    }
    if (one) atomicAdd(&cnt[p.E], 1);
    if (p.router == 2) {
      // ntlb: one density per pass, every token's top_k candidates
      // (moe.py:839-847); the probabilities and the repeated first-arg-max are
      // those of the forward kernel, so the candidates are the same
      const float* row = logits + t * p.E;
      const bool bf = p.softmax_bf16 != 0;
      const float neglse = -gb_logsumexp(row, p.E, bf);
      int ids[GB_MAX_K];
#pragma unroll
      for (int i = 0; i < GB_MAX_K; ++i) {
        if (i < p.top_k) {
          float best = -1.f;
          int bi = 0;
          for (int e = 0; e < p.E; ++e) {
            bool taken = false;
#pragma unroll
            for (int j = 0; j < GB_MAX_K; ++j) taken |= (j < i && ids[j] == e);
            const float v = taken ? -2.f : gb_prob(row[e], neglse, bf);
            if (v > best) { best = v; bi = e; }
          }
          ids[i] = bi;
          atomicAdd(&cnt[bi], 1);
        }
      }
      continue;
    }
    // top-2: density_1 counts mask_1 after the importance mask
    // (moe.py:1402-1420); switch: every token's arg-max (moe.py:1224)
    if (one || p.router == 1) atomicAdd(&cnt[idx[t * 2]], 1);
    // density_2 counts mask_2 = one_hot(index_2) * (importance > 0), before
    // the second-choice policy and the capacity (moe.py:1409-1411, :1429)
    if (p.use_second_place_loss && positive)
      atomicAdd(&cnt2[idx[t * 2 + 1]], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < p.E; e += blockDim.x) {
    if (cnt[e]) atomicAdd(&counts[(int64_t)g * p.E + e], cnt[e]);
    if (cnt2[e]) atomicAdd(&counts[((int64_t)p.G + g) * p.E + e], cnt2[e]);
  }
  if (threadIdx.x == 0 && cnt[p.E]) atomicAdd(&n_one[g], (float)cnt[p.E]);
}

template <typename IT>
__global__ __launch_bounds__(256) void gating_backward_kernel(
    GateBackwardParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, const int32_t* __restrict__ idx,
    const uint8_t* __restrict__ kept, const float* __restrict__ dgate,
    const float* __restrict__ d_loss, const int32_t* __restrict__ counts,
    const float* __restrict__ n_one, float* __restrict__ dlogits,
    int staged) {
  // staged: the block's rows of logits go through LDS (whole-line loads, rows
  // padded by one float against bank conflicts), the thread works on its row
  // there in place, and the rows of d(logits) leave the same way.  A thread
  // reading its 4 E bytes straight from global memory waits for a cache line
  // in every trip of every pass over the row.
  extern __shared__ __attribute__((aligned(16))) float gb_tile[];
  const int E = p.E, S = p.S;
  const int64_t T_tokens = (int64_t)p.G * p.S;
  const int64_t t_blk = (int64_t)blockIdx.x * blockDim.x;
  const int64_t t = t_blk + threadIdx.x;
  const int n_rows = (int)min((int64_t)blockDim.x, T_tokens - t_blk);
  if (staged) {
    const float* src = logits + t_blk * E;
    for (int q = threadIdx.x; q < n_rows * E; q += blockDim.x)
      gb_tile[(q / E) * (E + 1) + q % E] = src[q];
    __syncthreads();
  }
  if (t < T_tokens) {
  const int g = (int)(t / S);
  const float* row = staged ? gb_tile + threadIdx.x * (E + 1) : logits + t * E;
  float* out = staged ? gb_tile + threadIdx.x * (E + 1) : dlogits + t * E;
  // softmax exactly as the forward kernel computes it
  const bool bf = p.softmax_bf16 != 0;
  const float lse = gb_logsumexp(row, E, bf);
  const float neglse = -lse;
  float m1 = 1.0f;
  if (importance != nullptr) {
    const float imp = load_f32<IT>(importance + t);
    m1 = (p.importance_from_slot_gate ? imp > 0.5f : imp == 1.0f) ? 1.0f : 0.0f;
  }
  const int i1 = idx[t * 2], i2 = idx[t * 2 + 1];
  const float k1 = kept[t * 2] ? 1.0f : 0.0f, k2 = kept[t * 2 + 1] ? 1.0f : 0.0f;
  const float mb =
      p.num_microbatches > 1 ? (float)(1.0 / (double)p.num_microbatches) : 1.0f;
  const float dl = d_loss[0] * p.loss_scale;
  const float inv_s = (float)(1.0 / (double)S);
  const float ee = (float)((double)E * (double)E);
  float add1 = 0.f, add2 = 0.f;  // d(p[i1]), d(p[i2]) from the gates
  float coef;                    // d(p[e]) = coef * counts[g,e] from the loss
  if (p.router == 0) {
    const float p1 = gb_prob(row[i1], neglse, bf);
    const float p2 = gb_prob(row[i2], neglse, bf);
    const float g1 = p1 * m1;
    const float same = (i2 == i1) ? m1 : 0.0f;
    const float g2 = p2 * (1.0f - same);
    const float dg1n = dgate[t * 2] * k1, dg2n = dgate[t * 2 + 1] * k2;
    const float rec = 1.0f / ((g1 + g2) + 1e-9f);
    const float common = (dg1n * g1 + dg2n * g2) * rec * rec;
    add1 = (dg1n * rec - common) * m1;
    add2 = (dg2n * rec - common) * (1.0f - same);
    // loss = mean_{g,e}(mean_s(p * m1) * density_1) * E^2, density = count / S
    coef = dl * mb * ee * (float)(1.0 / ((double)p.G * (double)E)) * inv_s *
           inv_s * m1;
  } else {
    // switch: the gate is the arg-max probability; ntlb: the probability of
    // the candidate that took the token, and the loss averages over the
    // top_k passes as well (moe.py:845-856)
    add1 = dgate[t * 2] * k1 * m1;
    const double terms =
        (double)p.G * (double)E * (p.router == 2 ? (double)p.top_k : 1.0);
    if (p.has_importance)
      coef = dl * mb * ee * (float)(1.0 / (terms * (double)S)) * n_one[g] *
             inv_s * inv_s;
    else
      coef = dl * mb * ee * (float)(1.0 / terms) * inv_s * inv_s;
  }
  const int32_t* cg = counts + (int64_t)g * E;
  // Second-place loss (moe.py:1426-1438): 0.5 * E^2 * mean_{g,e}(mean_s(n) *
  // density_2) with n = q / (sum(q) + 1e-9), q = p * (1 - mask_1):
  // d/dq[e] = c2[e] * rq - (sum_f c2[f] q[f]) * rq^2, c2 = coef2 * count_2.
  const int32_t* cg2 = counts + ((int64_t)p.G + g) * E;
  const bool loss2 = p.router == 0 && p.use_second_place_loss;
  float coef2 = 0.f, rq = 0.f, aq = 0.f;
  if (loss2) {
    coef2 = dl * mb * 0.5f * ee * (float)(1.0 / ((double)p.G * (double)E)) *
            inv_s * inv_s;
    float q = 0.f, a = 0.f;
    for (int e = 0; e < E; ++e) {
      const float qe =
          gb_prob(row[e], neglse, bf) * (e == i1 ? 1.0f - m1 : 1.0f);
      q += qe;
      a += coef2 * (float)cg2[e] * qe;
    }
    rq = 1.0f / (q + 1e-9f);
    aq = a * rq * rq;
  }
  auto dprob = [&](int e) {
    float dp = coef * (float)cg[e];
    if (e == i1) dp += add1;
    if (p.router == 0 && e == i2) dp += add2;
    if (loss2)
      dp += (e == i1 ? 1.0f - m1 : 1.0f) * (coef2 * (float)cg2[e] * rq - aq);
    return dp;
  };
  // inner = sum_e p[e] * dp[e]
  float inner = 0.f;
  for (int e = 0; e < E; ++e) inner += gb_prob(row[e], neglse, bf) * dprob(e);
  float zfac = 0.f;
  if (p.use_z_loss) {  // d/dx of z_coef * sum(lse^2 * m1) / (n * microbatches)
    float n = 0.f;
    for (int gg = 0; gg < p.G; ++gg) n += n_one[gg];
    const float mbz = (float)(p.num_microbatches > 0 ? p.num_microbatches : 1);
    zfac = (d_loss[0] * p.loss_scale * p.z_loss_coef * 2.0f) * lse * m1 /
           (n * mbz);
  }
  for (int e = 0; e < E; ++e) {
    const float pe = gb_prob(row[e], neglse, bf);
    out[e] = pe * (dprob(e) - inner) + zfac * pe;
  }
  }  // t < T_tokens
  if (staged) {
    __syncthreads();
    float* dst = dlogits + t_blk * E;
    for (int q = threadIdx.x; q < n_rows * E; q += blockDim.x)
      dst[q] = gb_tile[(q / E) * (E + 1) + q % E];
  }
}

// ---------------------------------------------------------------------------
// The same product on the float32 matrix cores (v_mfma_f32_32x32x2_f32: two
// tokens per instruction, lanes 0-31 bring the first, lanes 32-63 the second;
// x as the row operand, dlogits as the column operand, both read as they lie
// in memory).  Block = 128 kernel rows x 64 experts x 512 tokens, 32 tokens
// staged in LDS at a time as float32 (rows padded by 32 floats so that the two
// half-waves hit different banks); a wavefront owns 32 rows x 64 experts.
// Needs M % 128 == 0, E % 8 == 0 and 16-byte aligned rows.
// ---------------------------------------------------------------------------
constexpr int WM_M = 128, WM_TOK = 512, WM_KT = 32;
typedef float wm_f32x16_t __attribute__((ext_vector_type(16)));

template <typename T>
__global__ __launch_bounds__(256) void router_wgrad_mfma_kernel(
    const T* __restrict__ x, const float* __restrict__ dlogits,
    float* __restrict__ acc_out, int64_t T_tokens, int M, int E) {
  constexpr int VN = Vec16B<T>::N;            // elements per 16-byte piece
  __shared__ float xs[WM_KT][WM_M + 32];
  __shared__ float ds[WM_KT][64 + 32];
  const int m0 = blockIdx.x * WM_M, e0 = blockIdx.z * 64;
  const int64_t t0 = (int64_t)blockIdx.y * WM_TOK;
  const int64_t t1 = t0 + WM_TOK < T_tokens ? t0 + WM_TOK : T_tokens;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  wm_f32x16_t acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
  // staging: thread -> (token row tid / 8, 16 kernel rows / 8 experts)
  const int sr = tid >> 3, sc = tid & 7;
  for (int64_t tb = t0; tb < t1; tb += WM_KT) {
    const int64_t t = tb + sr;
    float xv[16], dv[8];
    if (t < t1) {
      const T* xp = x + t * M + m0 + sc * 16;
#pragma unroll
      for (int u = 0; u < 16 / VN; ++u) {
        float f[VN];
        unpack16(*reinterpret_cast<const uint4*>(xp + u * VN), f, T());
#pragma unroll
        for (int j = 0; j < VN; ++j) xv[u * VN + j] = f[j];
      }
      if (e0 + sc * 8 < E) {
        const float4 a = *reinterpret_cast<const float4*>(dlogits + t * E + e0 + sc * 8);
        const float4 b = *reinterpret_cast<const float4*>(dlogits + t * E + e0 + sc * 8 + 4);
        dv[0] = a.x; dv[1] = a.y; dv[2] = a.z; dv[3] = a.w;
        dv[4] = b.x; dv[5] = b.y; dv[6] = b.z; dv[7] = b.w;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) dv[j] = 0.f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 16; ++j) xv[j] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) dv[j] = 0.f;
    }
    __syncthreads();                 // the previous batch has been consumed
#pragma unroll
    for (int j = 0; j < 16; j += 4)
      *reinterpret_cast<float4*>(&xs[sr][sc * 16 + j]) =
          make_float4(xv[j], xv[j + 1], xv[j + 2], xv[j + 3]);
    *reinterpret_cast<float4*>(&ds[sr][sc * 8]) = make_float4(dv[0], dv[1], dv[2], dv[3]);
    *reinterpret_cast<float4*>(&ds[sr][sc * 8 + 4]) = make_float4(dv[4], dv[5], dv[6], dv[7]);
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < WM_KT / 2; ++ks) {
      const float a = xs[2 * ks + half][wave * 32 + l32];
      const float b0 = ds[2 * ks + half][l32];
      const float b1 = ds[2 * ks + half][32 + l32];
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b0, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b1, acc1, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + wave * 32 + 8 * (r / 4) + 4 * half + (r % 4);
    if (e0 + l32 < E) atomicAdd(acc_out + (int64_t)m * E + e0 + l32, acc0[r]);
    if (e0 + 32 + l32 < E)
      atomicAdd(acc_out + (int64_t)m * E + e0 + 32 + l32, acc1[r]);
  }
}

// ---------------------------------------------------------------------------
// The same product for bfloat16 tokens on the bfloat16 matrix cores
// (v_mfma_f32_32x32x16_bf16, 16 tokens per instruction instead of 2).  The
// float32 d(logits) go in as two bfloat16 terms, hi = bf16(d) and
// lo = bf16(d - hi): x * hi and x * lo are exact in the float32 accumulator and
// what is left of d, at most 2^-17 |d|, is below the rounding of the sum
// itself.  Both operands lie in memory with the reduction index (the token)
// outermost; they are staged in LDS as they lie and the instruction's
// operands (8 consecutive tokens of one kernel row / one expert per lane) are
// read with ds_read_b64_tr_b16: within 16 lanes, lane t addresses the 8 bytes
// at (row t / 4, elements 4 (t % 4) ..) of a 4 x 16 block and lane i receives
// the block's column i.  Block = 128 kernel rows x 64 experts x WB_TOK tokens,
// 32 tokens staged at a time; a wavefront owns 32 rows x 64 experts.  Rows are
// padded so that the four rows of a block lie in different banks.  Every
// block writes its sums to its token chunk's [M, E] plane of the workspace
// and router_wgrad_reduce_kernel adds the planes in chunk order: the same
// bits on every run (the other kernels add with float atomics).
// Needs M % 128 == 0, E % 8 == 0 and 16-byte aligned rows.
// ---------------------------------------------------------------------------
constexpr int WB_M = 128, WB_TOK = 2048, WB_KT = 32;
constexpr int WB_XS = (WB_M + 32) * 2;   // bytes per staged token row of x
constexpr int WB_DS = (64 + 16) * 2;     // ... of one half of d(logits)
typedef __attribute__((ext_vector_type(8))) __bf16 wb_bf16x8_t;
typedef short wb_i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void wb_lds_void_t;

// 8 consecutive rows of this lane's column: rows 0-3 of the block at byte
// offset OFF from addr, rows 4-7 at OFF + ROW4
template <int OFF, int ROW4>
__device__ __forceinline__ wb_bf16x8_t lds_read_tr8(uint32_t addr) {
  wb_i16x4_t lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(lo) : "v"(addr), "n"(OFF) : "memory");
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(hi) : "v"(addr), "n"(OFF + ROW4) : "memory");
  return __builtin_bit_cast(
      wb_bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

__global__ __launch_bounds__(256) void router_wgrad_bf16_kernel(
    const bf16_t* __restrict__ x, const float* __restrict__ dlogits,
    float* __restrict__ acc_out, int64_t T_tokens, int M, int E) {
  __shared__ __attribute__((aligned(16))) unsigned char xs[WB_KT * WB_XS];
  __shared__ __attribute__((aligned(16))) unsigned char dhs[WB_KT * WB_DS];
  __shared__ __attribute__((aligned(16))) unsigned char dls[WB_KT * WB_DS];
  const int m0 = blockIdx.x * WB_M, e0 = blockIdx.z * 64;
  const int64_t t0 = (int64_t)blockIdx.y * WB_TOK;
  const int64_t t1 = t0 + WB_TOK < T_tokens ? t0 + WB_TOK : T_tokens;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  wm_f32x16_t acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
  // staging: thread -> (token row tid / 8, 16 kernel rows / 8 experts)
  const int sr = tid >> 3, sc = tid & 7;
  // transposed reads: this lane's row and first column within a 16 x 32 block
  const int t16 = lane & 15, g16 = lane >> 4;
  const int rrow = (g16 >> 1) * 8 + (t16 >> 2);
  const int rcol = (g16 & 1) * 16 + 4 * (t16 & 3);
  const uint32_t xa = (uint32_t)(size_t)(wb_lds_void_t*)xs + rrow * WB_XS +
                      (wave * 32 + rcol) * 2;
  const uint32_t ha = (uint32_t)(size_t)(wb_lds_void_t*)dhs + rrow * WB_DS +
                      rcol * 2;
  const uint32_t la = (uint32_t)(size_t)(wb_lds_void_t*)dls + rrow * WB_DS +
                      rcol * 2;
  const uint4 z4 = make_uint4(0, 0, 0, 0);
  for (int64_t tb = t0; tb < t1; tb += WB_KT) {
    const int64_t t = tb + sr;
    uint4 xv0 = z4, xv1 = z4, dh = z4, dl = z4;
    if (t < t1) {
      const uint4* xp = reinterpret_cast<const uint4*>(x + t * M + m0 + sc * 16);
      xv0 = xp[0];
      xv1 = xp[1];
      if (e0 + sc * 8 < E) {
        const float4 a = *reinterpret_cast<const float4*>(dlogits + t * E + e0 + sc * 8);
        const float4 b = *reinterpret_cast<const float4*>(dlogits + t * E + e0 + sc * 8 + 4);
        const float d[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        float lo[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) lo[j] = d[j] - round_to<bf16_t>(d[j]);
        dh = pack16(d, bf16_t());
        dl = pack16(lo, bf16_t());
      }
    }
    __syncthreads();                 // the previous batch has been consumed
    *reinterpret_cast<uint4*>(xs + sr * WB_XS + sc * 32) = xv0;
    *reinterpret_cast<uint4*>(xs + sr * WB_XS + sc * 32 + 16) = xv1;
    *reinterpret_cast<uint4*>(dhs + sr * WB_DS + sc * 16) = dh;
    *reinterpret_cast<uint4*>(dls + sr * WB_DS + sc * 16) = dl;
    __syncthreads();
    // 16 tokens per step: the x operand and, per 32 experts, hi and lo
    const wb_bf16x8_t a0 = lds_read_tr8<0, 4 * WB_XS>(xa);
    const wb_bf16x8_t h00 = lds_read_tr8<0, 4 * WB_DS>(ha);
    const wb_bf16x8_t l00 = lds_read_tr8<0, 4 * WB_DS>(la);
    const wb_bf16x8_t h01 = lds_read_tr8<64, 4 * WB_DS>(ha);
    const wb_bf16x8_t l01 = lds_read_tr8<64, 4 * WB_DS>(la);
    const wb_bf16x8_t a1 = lds_read_tr8<16 * WB_XS, 4 * WB_XS>(xa);
    const wb_bf16x8_t h10 = lds_read_tr8<16 * WB_DS, 4 * WB_DS>(ha);
    const wb_bf16x8_t l10 = lds_read_tr8<16 * WB_DS, 4 * WB_DS>(la);
    const wb_bf16x8_t h11 = lds_read_tr8<16 * WB_DS + 64, 4 * WB_DS>(ha);
    const wb_bf16x8_t l11 = lds_read_tr8<16 * WB_DS + 64, 4 * WB_DS>(la);
    // the compiler does not count the asm reads: wait for them here
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, h00, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, h01, acc1, 0, 0, 0);
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, l00, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, l01, acc1, 0, 0, 0);
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, h10, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, h11, acc1, 0, 0, 0);
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, l10, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, l11, acc1, 0, 0, 0);
  }
  // this block's partial sums: chunk blockIdx.y of acc_out [chunks][M][E]
  float* part = acc_out + (int64_t)blockIdx.y * M * E;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + wave * 32 + 8 * (r / 4) + 4 * half + (r % 4);
    if (e0 + l32 < E) part[(int64_t)m * E + e0 + l32] = acc0[r];
    if (e0 + 32 + l32 < E) part[(int64_t)m * E + e0 + 32 + l32] = acc1[r];
  }
}

// dw = sum over the token chunks of the partial sums, in chunk order
template <typename T>
__global__ void router_wgrad_reduce_kernel(const float* __restrict__ part,
                                           T* __restrict__ dw, int64_t n,
                                           int chunks) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float sum = 0.f;
  for (int c = 0; c < chunks; ++c) sum += part[(int64_t)c * n + i];
  store_f32<T>(dw + i, sum);
}

// ---------------------------------------------------------------------------
// router projection backward w.r.t. the kernel: dw[m,e] = sum_t x[t,m] *
// dlogits[t,e], float32.  Block (m tile of 256, chunk of tokens, chunk of 64
// experts) accumulates 256 x 64 partial sums and adds them to the float32
// accumulator with atomics.  Thread (m group = tid % 64, expert group =
// tid / 64) owns a 4 x 16 patch: per staged token one 16-byte LDS read of x
// and four (broadcast) of dlogits feed 64 multiply-adds.
// ---------------------------------------------------------------------------
constexpr int WG_TOK = 1024;  // tokens per block
constexpr int WG_BATCH = 32;  // tokens staged in LDS at a time
constexpr int WG_M = 256;     // kernel rows per block

template <typename T>
__global__ __launch_bounds__(256) void router_wgrad_kernel(
    const T* __restrict__ x, const float* __restrict__ dlogits,
    float* __restrict__ acc_out, int64_t T_tokens, int M, int E, bool vec) {
  __shared__ __attribute__((aligned(16))) float xs[WG_BATCH][WG_M];
  __shared__ __attribute__((aligned(16))) float ds[WG_BATCH][64];
  const int m0 = blockIdx.x * WG_M, e0 = blockIdx.z * 64;
  const int64_t t0 = (int64_t)blockIdx.y * WG_TOK;
  const int64_t t1 = t0 + WG_TOK < T_tokens ? t0 + WG_TOK : T_tokens;
  const int tid = threadIdx.x;
  const int mg = tid & 63, eg = tid >> 6;  // rows m0 + 4 mg .., experts e0 + 16 eg ..
  float acc[4][16];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  for (int64_t tb = t0; tb < t1; tb += WG_BATCH) {
    if (vec) {
      // 16-byte pieces, all of a thread's loads in flight before the first
      // LDS write
      constexpr int VN = Vec16B<T>::N;
      constexpr int XP = WG_BATCH * WG_M / VN / 256;   // pieces of x per thread
      uint4 xv[XP];
      float4 dv[2];
#pragma unroll
      for (int u = 0; u < XP; ++u) {
        const int i = tid + u * 256;
        const int r = i / (WG_M / VN), c = (i % (WG_M / VN)) * VN;
        const int64_t t = tb + r;
        xv[u] = (t < t1 && m0 + c < M)
                    ? *reinterpret_cast<const uint4*>(x + t * M + m0 + c)
                    : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int i = tid + u * 256;
        const int r = i >> 4, c = (i & 15) * 4;
        const int64_t t = tb + r;
        dv[u] = (t < t1 && e0 + c < E)
                    ? *reinterpret_cast<const float4*>(dlogits + t * E + e0 + c)
                    : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < XP; ++u) {
        const int i = tid + u * 256;
        const int r = i / (WG_M / VN), c = (i % (WG_M / VN)) * VN;
        float f[VN];
        unpack16(xv[u], f, T());
#pragma unroll
        for (int q = 0; q < VN; ++q) xs[r][c + q] = f[q];
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int i = tid + u * 256;
        *reinterpret_cast<float4*>(&ds[i >> 4][(i & 15) * 4]) = dv[u];
      }
    } else {
      for (int i = tid; i < WG_BATCH * WG_M; i += 256) {
        const int r = i / WG_M, c = i % WG_M;
        const int64_t t = tb + r;
        xs[r][c] = (t < t1 && m0 + c < M) ? load_f32<T>(x + t * M + m0 + c) : 0.f;
      }
      for (int i = tid; i < WG_BATCH * 64; i += 256) {
        const int r = i >> 6, c = i & 63;
        const int64_t t = tb + r;
        ds[r][c] = (t < t1 && e0 + c < E) ? dlogits[t * E + e0 + c] : 0.f;
      }
    }
    __syncthreads();
#pragma unroll 2
    for (int r = 0; r < WG_BATCH; ++r) {
      const float4 xv = *reinterpret_cast<const float4*>(&xs[r][mg * 4]);
      const float xa[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 dv = *reinterpret_cast<const float4*>(&ds[r][eg * 16 + q * 4]);
        const float da[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][q * 4 + j] = fmaf(xa[i], da[j], acc[i][q * 4 + j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + mg * 4 + i;
    if (m < M) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int e = e0 + eg * 16 + j;
        if (e < E) atomicAdd(acc_out + (int64_t)m * E + e, acc[i][j]);
      }
    }
  }
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride)
    p[i] = v;
}

template <typename T>
__global__ void convert_f32_kernel(const float* src, T* dst, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride)
    store_f32<T>(dst + i, src[i]);
}

static bool bw_aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// dx = rows of dexpert_in named by tok_slot + dlogits . w_gate^T through
// dispatch_backward_mfma_kernel<.., SLOT>; false if the kernel does not take
// the case (nothing launched).
bool launch_slot_dispatch_backward_mfma(
    const void* dexpert_in, const int16_t* tok_slot, const float* dlogits,
    const void* w_gate, void* dx, int G, int S, int E, int C, int M, int dtype,
    hipStream_t st, int* rc) {
  const int64_t T_tokens = (int64_t)G * S;
  *rc = 0;
  if (!(dtype == MESH_MOE_BF16 && dlogits != nullptr && w_gate != nullptr &&
        bw_aligned16(dexpert_in) && bw_aligned16(dx) && bw_aligned16(w_gate) &&
        bw_aligned16(dlogits) && E % 16 == 0 && E <= DBM_MAX_E &&
        M % DBM_COLS == 0 && S % DBM_TOK == 0 &&
        (T_tokens + DBM_TOK - 1) / DBM_TOK <= 65535))
    return false;
  dim3 grid((unsigned)(M / DBM_COLS),
            (unsigned)((T_tokens + DBM_TOK - 1) / DBM_TOK));
  const size_t lds = dbm_lds_bytes(E);
  auto run = [&](auto k) -> int {
    MOE_ALLOW_LDS(k, lds);
    k<<<grid, 256, lds, st>>>(
        (const bf16_t*)dexpert_in, nullptr, nullptr, nullptr, nullptr, dlogits,
        (const bf16_t*)w_gate, (bf16_t*)dx, G, S, C, M, T_tokens, G, nullptr,
        tok_slot);
    MOE_CHECK_LAUNCH("slot_dispatch_backward (router share on the matrix cores)");
    return 0;
  };
  switch (E / 16) {
    case 1: *rc = run(dispatch_backward_mfma_kernel<1, true>); break;
    case 2: *rc = run(dispatch_backward_mfma_kernel<2, true>); break;
    case 3: *rc = run(dispatch_backward_mfma_kernel<3, true>); break;
    case 4: *rc = run(dispatch_backward_mfma_kernel<4, true>); break;
    case 5: *rc = run(dispatch_backward_mfma_kernel<5, true>); break;
    case 6: *rc = run(dispatch_backward_mfma_kernel<6, true>); break;
    case 7: *rc = run(dispatch_backward_mfma_kernel<7, true>); break;
    default: *rc = run(dispatch_backward_mfma_kernel<8, true>); break;
  }
  return true;
}

}  // namespace mesh_moe

using namespace mesh_moe;

static int run_combine_backward(
    const void* dout, const void* y, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* fill,
    const int32_t* row_offsets, void* dy, float* dgate, int G, int S, int E,
    int C, int N, int dtype, void* stream);

extern "C" int mesh_moe_combine_backward(
    const void* dout, const void* y, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* fill, void* dy,
    float* dgate, int G, int S, int E, int C, int N, int dtype, void* stream) {
  return run_combine_backward(dout, y, idx, pos, gate, kept, fill, nullptr, dy,
                              dgate, G, S, E, C, N, dtype, stream);
}

extern "C" int mesh_moe_combine_backward_compact(
    const void* dout, const void* y, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* fill,
    const int32_t* row_offsets, void* dy, float* dgate, int G, int S, int E,
    int C, int N, int dtype, void* stream) {
  MOE_REQUIRE(row_offsets, MESH_MOE_E_ARG,
              "combine_backward_compact: null pointer");
  return run_combine_backward(dout, y, idx, pos, gate, kept, fill, row_offsets,
                              dy, dgate, G, S, E, C, N, dtype, stream);
}

static int run_combine_backward(
    const void* dout, const void* y, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* fill,
    const int32_t* row_offsets, void* dy, float* dgate, int G, int S, int E,
    int C, int N, int dtype, void* stream) {
  MOE_REQUIRE(dout && y && idx && pos && gate && kept && fill && dy && dgate,
              MESH_MOE_E_ARG, "combine_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "combine_backward: bad dtype %d", dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && N >= 1, MESH_MOE_E_ARG,
              "combine_backward: bad sizes G=%d S=%d E=%d C=%d N=%d", G, S, E,
              C, N);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t njobs =
      T_tokens + (row_offsets != nullptr ? (int64_t)E * 256 : (int64_t)G * E);
  const int64_t nblocks = (njobs + BW_ROWS_PER_BLOCK - 1) / BW_ROWS_PER_BLOCK;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "combine_backward: too many rows (%lld)", (long long)njobs);
  const bool vec = ((size_t)N * dtype_size(dtype)) % 16 == 0 &&
                   bw_aligned16(dout) && bw_aligned16(y) && bw_aligned16(dy);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32)
    combine_backward_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)dout, (const float*)y, idx, pos, gate, kept, fill,
        (float*)dy, dgate, G, S, E, C, N, T_tokens, vec, row_offsets);
  else
    combine_backward_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)dout, (const bf16_t*)y, idx, pos, gate, kept, fill,
        (bf16_t*)dy, dgate, G, S, E, C, N, T_tokens, vec, row_offsets);
  MOE_CHECK_LAUNCH("combine_backward");
  return 0;
}

static int run_dispatch_backward(
    const void* dexpert_in, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* row_offsets,
    const float* dlogits, const void* w_gate_packed, const void* w_gate,
    int groups_per_router, void* dx, int G, int S, int E, int C, int M,
    int dtype, void* stream);

extern "C" int mesh_moe_dispatch_backward(
    const void* dexpert_in, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const float* dlogits,
    const void* w_gate_packed, const void* w_gate, int groups_per_router,
    void* dx, int G, int S, int E, int C, int M, int dtype, void* stream) {
  return run_dispatch_backward(dexpert_in, idx, pos, gate, kept, nullptr,
                               dlogits, w_gate_packed, w_gate,
                               groups_per_router, dx, G, S, E, C, M, dtype,
                               stream);
}

extern "C" int mesh_moe_dispatch_backward_compact(
    const void* dexpert_in, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* row_offsets,
    const float* dlogits, const void* w_gate_packed, const void* w_gate,
    int groups_per_router, void* dx, int G, int S, int E, int C, int M,
    int dtype, void* stream) {
  MOE_REQUIRE(row_offsets, MESH_MOE_E_ARG,
              "dispatch_backward_compact: null pointer");
  return run_dispatch_backward(dexpert_in, idx, pos, gate, kept, row_offsets,
                               dlogits, w_gate_packed, w_gate,
                               groups_per_router, dx, G, S, E, C, M, dtype,
                               stream);
}

static int run_dispatch_backward(
    const void* dexpert_in, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* row_offsets,
    const float* dlogits, const void* w_gate_packed, const void* w_gate,
    int groups_per_router, void* dx, int G, int S, int E, int C, int M,
    int dtype, void* stream) {
  MOE_REQUIRE(dexpert_in && idx && pos && gate && kept && dx, MESH_MOE_E_ARG,
              "dispatch_backward: null pointer");
  MOE_REQUIRE(w_gate_packed == nullptr ||
                  (groups_per_router >= 1 && G % groups_per_router == 0),
              MESH_MOE_E_ARG,
              "dispatch_backward: G=%d is not a multiple of "
              "groups_per_router=%d", G, groups_per_router);
  MOE_REQUIRE((dlogits == nullptr) == (w_gate_packed == nullptr),
              MESH_MOE_E_ARG,
              "dispatch_backward: dlogits and w_gate_packed go together");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "dispatch_backward: bad dtype %d", dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1, MESH_MOE_E_ARG,
              "dispatch_backward: bad sizes G=%d S=%d E=%d C=%d M=%d", G, S, E,
              C, M);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t nblocks =
      (T_tokens + BW_ROWS_PER_BLOCK - 1) / BW_ROWS_PER_BLOCK;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "dispatch_backward: too many rows (%lld)", (long long)T_tokens);
  const bool vec = ((size_t)M * dtype_size(dtype)) % 16 == 0 &&
                   bw_aligned16(dexpert_in) && bw_aligned16(dx) &&
                   (w_gate_packed == nullptr || bw_aligned16(w_gate_packed));
  hipStream_t st = (hipStream_t)stream;
  if (vec && dlogits != nullptr && w_gate != nullptr &&
      dtype == MESH_MOE_BF16 && bw_aligned16(w_gate) &&
      bw_aligned16(dlogits) && E % 16 == 0 && E <= DBM_MAX_E &&
      M % DBM_COLS == 0 && S % DBM_TOK == 0 &&
      (T_tokens + DBM_TOK - 1) / DBM_TOK <= 65535) {
    dim3 grid((unsigned)(M / DBM_COLS),
              (unsigned)((T_tokens + DBM_TOK - 1) / DBM_TOK));
    const size_t lds = dbm_lds_bytes(E);
#define MOE_DBM(KS_)                                                         \
  do {                                                                       \
    auto k = row_offsets != nullptr                                          \
                 ? dispatch_backward_mfma_kernel<KS_, false, true>           \
                 : dispatch_backward_mfma_kernel<KS_, false, false>;         \
    MOE_ALLOW_LDS(k, lds);                                                   \
    k<<<grid, 256, lds, st>>>(                                               \
        (const bf16_t*)dexpert_in, idx, pos, gate, kept, dlogits,            \
        (const bf16_t*)w_gate, (bf16_t*)dx, G, S, C, M, T_tokens,            \
        groups_per_router, row_offsets, nullptr);                            \
  } while (0)
    switch (E / 16) {
      case 1: MOE_DBM(1); break;
      case 2: MOE_DBM(2); break;
      case 3: MOE_DBM(3); break;
      case 4: MOE_DBM(4); break;
      case 5: MOE_DBM(5); break;
      case 6: MOE_DBM(6); break;
      case 7: MOE_DBM(7); break;
      default: MOE_DBM(8); break;
    }
#undef MOE_DBM
    MOE_CHECK_LAUNCH("dispatch_backward (router share on the matrix cores)");
    return 0;
  }
  if (vec && dlogits != nullptr && E <= DBR_MAX_E && S % DBR_TOK == 0) {
    const int64_t nb4 = (T_tokens + 4 * DBR_TOK - 1) / (4 * DBR_TOK);
    if (dtype == MESH_MOE_F32)
      dispatch_backward_router4_kernel<float><<<(unsigned)nb4, 256, 0, st>>>(
          (const float*)dexpert_in, idx, pos, gate, kept, dlogits,
          (const float*)w_gate_packed, (float*)dx, G, S, E, C, M, T_tokens,
          groups_per_router, row_offsets);
    else
      dispatch_backward_router4_kernel<bf16_t><<<(unsigned)nb4, 256, 0, st>>>(
          (const bf16_t*)dexpert_in, idx, pos, gate, kept, dlogits,
          (const bf16_t*)w_gate_packed, (bf16_t*)dx, G, S, E, C, M, T_tokens,
          groups_per_router, row_offsets);
    MOE_CHECK_LAUNCH("dispatch_backward (router share, 4 tokens per wavefront)");
    return 0;
  }
  if (dtype == MESH_MOE_F32)
    dispatch_backward_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)dexpert_in, idx, pos, gate, kept, dlogits,
        (const float*)w_gate_packed, (float*)dx, G, S, E, C, M, T_tokens,
        groups_per_router, vec, row_offsets);
  else
    dispatch_backward_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)dexpert_in, idx, pos, gate, kept, dlogits,
        (const bf16_t*)w_gate_packed, (bf16_t*)dx, G, S, E, C, M, T_tokens,
        groups_per_router, vec, row_offsets);
  MOE_CHECK_LAUNCH("dispatch_backward");
  return 0;
}

extern "C" size_t mesh_moe_gating_backward_workspace_bytes(int G, int E) {
  if (G < 1 || E < 1) return 0;
  // counts of first and of second choices [2][G][E], tokens of importance 1 [G]
  return sizeof(int32_t) * 2 * (size_t)G * E + sizeof(float) * (size_t)G + 256;
}

extern "C" int mesh_moe_gating_backward(
    const float* logits, const void* importance, int importance_dtype,
    int importance_from_slot_gate, const int32_t* idx, const uint8_t* kept,
    const float* dgate, const float* d_loss, double loss_scale, int G, int S,
    int E, int router, int top_k, int softmax_dtype, int use_second_place_loss,
    int use_z_loss, double z_loss_coef, int num_microbatches, float* dlogits,
    void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && idx && kept && dgate && d_loss && dlogits && workspace,
              MESH_MOE_E_ARG, "gating_backward: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 2 && E <= 512 && G <= 65535,
              MESH_MOE_E_ARG, "gating_backward: bad sizes G=%d S=%d E=%d", G, S,
              E);
  MOE_REQUIRE(router >= 0 && router <= 2, MESH_MOE_E_ARG,
              "gating_backward: unknown router %d", router);
  MOE_REQUIRE(router != 2 || (top_k >= 1 && top_k <= E && top_k <= GB_MAX_K),
              MESH_MOE_E_ARG, "gating_backward: top_k=%d with %d experts "
              "(at most %d)", top_k, E, GB_MAX_K);
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "gating_backward: bad importance dtype %d", importance_dtype);
  MOE_REQUIRE(valid_dtype(softmax_dtype), MESH_MOE_E_ARG,
              "gating_backward: bad softmax dtype %d", softmax_dtype);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_gating_backward_workspace_bytes(G, E),
              MESH_MOE_E_ARG, "gating_backward: workspace too small");
  GateBackwardParams p;
  p.G = G; p.S = S; p.E = E;
  p.router = router;
  p.top_k = top_k;
  p.use_second_place_loss = (use_second_place_loss && router == 0) ? 1 : 0;
  p.has_importance = importance != nullptr;
  p.importance_from_slot_gate = importance_from_slot_gate ? 1 : 0;
  p.num_microbatches = num_microbatches;
  p.use_z_loss = (use_z_loss && router == 1) ? 1 : 0;
  p.z_loss_coef = (float)z_loss_coef;
  p.loss_scale = (float)loss_scale;
  // only _ntlb_gating runs its softmax in the activation dtype
  p.softmax_bf16 = (router == 2 && softmax_dtype == MESH_MOE_BF16) ? 1 : 0;
  uintptr_t wsp = ((uintptr_t)workspace + 255) & ~(uintptr_t)255;
  int32_t* counts = (int32_t*)wsp;
  float* n_one = (float*)(counts + 2 * (size_t)G * E);
  hipStream_t st = (hipStream_t)stream;
  const size_t smem = sizeof(int32_t) * (2 * (size_t)E + 1);
  const int64_t T_tokens = (int64_t)G * S;
  // rows through LDS where a block's rows fit: 256 threads up to 64 experts,
  // 128 threads up to 128
  const int staged = E <= 128;
  const unsigned gb_threads = (staged && E > 64) ? 128 : 256;
  const size_t gb_smem = staged ? sizeof(float) * gb_threads * (E + 1) : 0;
  const unsigned blocks =
      (unsigned)((T_tokens + gb_threads - 1) / gb_threads);
  // the counters (int32 counts, then float n_one: all-zero bits either way)
  const int64_t n_cnt = 2 * (int64_t)G * E + G;
  fill_f32_kernel<<<(unsigned)((n_cnt + 255) / 256 < 1024 ? (n_cnt + 255) / 256
                                                          : 1024),
                    256, 0, st>>>((float*)counts, n_cnt, 0.0f);
  MOE_CHECK_LAUNCH("gating_backward (clear)");
  // up to 16 blocks per group, 256 tokens or more each
  const dim3 cgrid((unsigned)G, (unsigned)((S + 255) / 256 < 16 ? (S + 255) / 256
                                                               : 16));
  if (importance && importance_dtype == MESH_MOE_BF16) {
    gate_count_kernel<bf16_t><<<cgrid, 256, smem, st>>>(
        p, logits, idx, (const bf16_t*)importance, counts, n_one);
    MOE_CHECK_LAUNCH("gating_backward (count)");
    auto k = gating_backward_kernel<bf16_t>;
    MOE_ALLOW_LDS(k, gb_smem);
    k<<<blocks, gb_threads, gb_smem, st>>>(
        p, logits, (const bf16_t*)importance, idx, kept, dgate, d_loss, counts,
        n_one, dlogits, staged);
  } else {
    gate_count_kernel<float><<<cgrid, 256, smem, st>>>(
        p, logits, idx, (const float*)importance, counts, n_one);
    MOE_CHECK_LAUNCH("gating_backward (count)");
    auto k = gating_backward_kernel<float>;
    MOE_ALLOW_LDS(k, gb_smem);
    k<<<blocks, gb_threads, gb_smem, st>>>(
        p, logits, (const float*)importance, idx, kept, dgate, d_loss, counts,
        n_one, dlogits, staged);
  }
  MOE_CHECK_LAUNCH("gating_backward");
  return 0;
}

static bool router_wgrad_bf16_applies(int64_t tokens, int M, int E, int dtype) {
  return dtype == MESH_MOE_BF16 && ((size_t)M * 2) % 16 == 0 && E % 8 == 0 &&
         M % WB_M == 0 && (tokens + WB_TOK - 1) / WB_TOK <= 65535;
}

extern "C" size_t mesh_moe_router_backward_weights_workspace_bytes(
    int64_t tokens, int M, int E, int dtype) {
  if (tokens < 1 || M < 1 || E < 1 || !valid_dtype(dtype)) return 0;
  const size_t planes = router_wgrad_bf16_applies(tokens, M, E, dtype)
                            ? (size_t)((tokens + WB_TOK - 1) / WB_TOK) : 1;
  return sizeof(float) * planes * (size_t)M * E;
}

extern "C" int mesh_moe_router_backward_weights(const void* x,
                                                const float* dlogits,
                                                void* dw_gate,
                                                float* workspace,
                                                int64_t tokens, int M, int E,
                                                int dtype, void* stream) {
  MOE_REQUIRE(x && dlogits && dw_gate && workspace, MESH_MOE_E_ARG,
              "router_backward_weights: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "router_backward_weights: bad dtype %d", dtype);
  MOE_REQUIRE(tokens >= 1 && M >= 1 && E >= 1, MESH_MOE_E_ARG,
              "router_backward_weights: bad sizes tokens=%lld M=%d E=%d",
              (long long)tokens, M, E);
  const int64_t chunks = (tokens + WG_TOK - 1) / WG_TOK;
  MOE_REQUIRE(chunks <= 65535 && (E + 63) / 64 <= 65535,
              MESH_MOE_E_UNSUPPORTED,
              "router_backward_weights: too many tokens (%lld)",
              (long long)tokens);
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = (int64_t)M * E;
  const unsigned fb = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (router_wgrad_bf16_applies(tokens, M, E, dtype) && bw_aligned16(x) &&
      bw_aligned16(dlogits)) {
    const int bchunks = (int)((tokens + WB_TOK - 1) / WB_TOK);
    dim3 bgrid((unsigned)(M / WB_M), (unsigned)bchunks,
               (unsigned)((E + 63) / 64));
    router_wgrad_bf16_kernel<<<bgrid, 256, 0, st>>>(
        (const bf16_t*)x, dlogits, workspace, tokens, M, E);
    MOE_CHECK_LAUNCH("router_backward_weights (mfma, bf16 terms)");
    router_wgrad_reduce_kernel<bf16_t><<<(unsigned)((n + 255) / 256), 256, 0,
                                         st>>>(workspace, (bf16_t*)dw_gate, n,
                                               bchunks);
    MOE_CHECK_LAUNCH("router_backward_weights (sum of the chunks)");
    return 0;
  }
  fill_f32_kernel<<<fb, 256, 0, st>>>(workspace, n, 0.0f);
  MOE_CHECK_LAUNCH("router_backward_weights (clear)");
  dim3 grid((unsigned)((M + WG_M - 1) / WG_M), (unsigned)chunks,
            (unsigned)((E + 63) / 64));
  // 16-byte loads: rows of x and of dlogits start 16-byte aligned and hold
  // whole pieces
  const bool vec = ((size_t)M * dtype_size(dtype)) % 16 == 0 && E % 4 == 0 &&
                   bw_aligned16(x) && bw_aligned16(dlogits);
  if (vec && M % WM_M == 0 && E % 8 == 0) {
    const int64_t mchunks = (tokens + WM_TOK - 1) / WM_TOK;
    MOE_REQUIRE(mchunks <= 65535, MESH_MOE_E_UNSUPPORTED,
                "router_backward_weights: too many tokens (%lld)",
                (long long)tokens);
    dim3 mgrid((unsigned)(M / WM_M), (unsigned)mchunks, (unsigned)((E + 63) / 64));
    if (dtype == MESH_MOE_F32) {
      router_wgrad_mfma_kernel<float><<<mgrid, 256, 0, st>>>(
          (const float*)x, dlogits, workspace, tokens, M, E);
      MOE_CHECK_LAUNCH("router_backward_weights (mfma)");
      convert_f32_kernel<float><<<fb, 256, 0, st>>>(workspace, (float*)dw_gate, n);
    } else {
      // (unaligned bf16 operands: the float32 matrix cores)
      router_wgrad_mfma_kernel<bf16_t><<<mgrid, 256, 0, st>>>(
          (const bf16_t*)x, dlogits, workspace, tokens, M, E);
      MOE_CHECK_LAUNCH("router_backward_weights (mfma)");
      convert_f32_kernel<bf16_t><<<fb, 256, 0, st>>>(workspace, (bf16_t*)dw_gate,
                                                    n);
    }
    MOE_CHECK_LAUNCH("router_backward_weights (convert)");
    return 0;
  }
  if (dtype == MESH_MOE_F32) {
    router_wgrad_kernel<float><<<grid, 256, 0, st>>>(
        (const float*)x, dlogits, workspace, tokens, M, E, vec);
    MOE_CHECK_LAUNCH("router_backward_weights");
    convert_f32_kernel<float><<<fb, 256, 0, st>>>(workspace, (float*)dw_gate, n);
  } else {
    router_wgrad_kernel<bf16_t><<<grid, 256, 0, st>>>(
        (const bf16_t*)x, dlogits, workspace, tokens, M, E, vec);
    MOE_CHECK_LAUNCH("router_backward_weights");
    convert_f32_kernel<bf16_t><<<fb, 256, 0, st>>>(workspace, (bf16_t*)dw_gate,
                                                  n);
  }
  MOE_CHECK_LAUNCH("router_backward_weights (convert)");
  return 0;
}
