// Router projection and top-2 gating (softmax, expert choice, capacity
// positions, balancing loss) for gfx950.
//
// Follows _top_2_gating, mesh_tensorflow/transformer/moe.py:1384-1496, with the
// float32 operation order of mtf.softmax (ops.py:5493-5541) and mtf.top_1
// (ops.py:4937-4940).  The dense [G,S,E] masks and the S x S cumsum matmul
// (ops.py:2761-2781) are replaced by a per-token record and integer counting.
#include <atomic>
#include <mutex>

#include "common.h"

namespace mesh_moe {

// ---------------------------------------------------------------------------
// Router logits: logits[b,t,e] = sum_m x[b,t,m] * w[b,m,e] (+ bias[e]).
// One block = 64 tokens; thread (tok = tid % 64, eg = tid / 64) accumulates
// experts eg*EPT .. eg*EPT+EPT-1 with EPT = ceil(E / 4) <= 32.  x and w are
// staged through LDS as float32 in chunks of KC columns of M.
// ---------------------------------------------------------------------------
constexpr int RL_TOK = 64;
constexpr int RL_KC = 64;
constexpr int RL_MAX_EPT = 32;

// EPT: experts per thread, a power of two >= ept (the loop over a thread's
// experts is unrolled without conditions: with EPT = 32 and a condition per
// expert the 64 x 32 scalar branches per chunk were the whole run time at
// E = 8; the surplus products read the next group's weights and are dropped)
template <typename T, int EPT>
__global__ __launch_bounds__(256) void router_logits_kernel(
    const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ bias, float* __restrict__ logits,
    int64_t tokens, int M, int E, int ept) {
  extern __shared__ float smem[];
  float* xs = smem;                       // [RL_TOK][RL_KC + 1]
  float* ws = smem + RL_TOK * (RL_KC + 1);  // [RL_KC][E] + 4 EPT
  const int b = blockIdx.y;
  const int64_t t0 = (int64_t)blockIdx.x * RL_TOK;
  const int tid = threadIdx.x;
  const int tok = tid & 63;
  const int eg = tid >> 6;
  const T* xb = x + ((int64_t)b * tokens) * M;
  const T* wb = w + (int64_t)b * M * E;
  float acc[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) acc[j] = 0.f;

  for (int k0 = 0; k0 < M; k0 += RL_KC) {
    // x tile: 64 tokens x KC, coalesced along M; a thread's 16 loads are all
    // issued before the first LDS write (one at a time, each waited for, the
    // staging took 30 us per chunk)
    float xv[RL_TOK * RL_KC / 256];
#pragma unroll
    for (int u = 0; u < RL_TOK * RL_KC / 256; ++u) {
      const int i = tid + u * 256;
      const int r = i / RL_KC, c = i % RL_KC;
      const int64_t t = t0 + r;
      xv[u] = (t < tokens && k0 + c < M) ? load_f32<T>(xb + t * M + k0 + c) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < RL_TOK * RL_KC / 256; ++u) {
      const int i = tid + u * 256;
      xs[(i / RL_KC) * (RL_KC + 1) + i % RL_KC] = xv[u];
    }
    for (int i = tid; i < RL_KC * E; i += 256) {
      int r = i / E, c = i % E;
      float v = 0.f;
      if (k0 + r < M) v = load_f32<T>(wb + (int64_t)(k0 + r) * E + c);
      ws[i] = v;
    }
    __syncthreads();
    const int e0 = eg * ept;
    for (int k = 0; k < RL_KC; ++k) {
      float xv = xs[tok * (RL_KC + 1) + k];
      const float* wr = ws + k * E + e0;
#pragma unroll
      for (int j = 0; j < EPT; ++j) acc[j] = fmaf(xv, wr[j], acc[j]);
    }
    __syncthreads();
  }
  int64_t t = t0 + tok;
  if (t < tokens) {
    float* out = logits + ((int64_t)b * tokens + t) * E;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      int e = eg * ept + j;
      if (j < ept && e < E) out[e] = bias ? acc[j] + bias[e] : acc[j];
    }
  }
}

// ---------------------------------------------------------------------------
// Router logits on the matrix cores (bf16 inputs, packed router weights
// wp[b][e][m]).  logits^T tile = wp tile (experts as MFMA rows) x x tile (tokens
// as MFMA columns): lane l ends up with token l % 32 of its wavefront and, per
// 32-expert tile, experts 8*(r/4) + 4*(l/32) + r%4 in accumulator register r.
// bf16 x bf16 products are exact in float32, so this is the float32 matmul of
// the reference on bf16-rounded operands up to summation order.
//
// A block is 4 wavefronts x 32 tokens; x and wp K tiles (64 deep) are brought
// into a three-slot LDS ring by global_load_lds_dwordx4 with the same
// 128-byte-row XOR swizzle as the expert GEMM.  The kernel is bound by reading
// x once from HBM.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 rl_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float rl_f32x16_t;
typedef __attribute__((address_space(3))) void rl_lds_void_t;
typedef const __attribute__((address_space(1))) void rl_glb_void_t;

// Cache-policy operand of the direct-to-LDS loads of the token tile: the
// non-temporal hint.  Every token row is read exactly once by these kernels;
// with the hint the fused router kernel runs 8 % faster (0.121 -> 0.112 ms at
// 65536 tokens x 4096).  The router weights keep the default policy: every
// block re-reads them from the L2.
constexpr int RL_STREAMING = 2;

__device__ __forceinline__ int rl_swizzle(int row) {
  return (row & 7) ^ ((row >> 3) & 1);
}

// Writes a block's 128 x E logits as whole rows.  The matrix cores leave a
// token's row spread over two lanes in groups of four experts (v[j][4 q + r]
// = expert 32 j + 8 q + 4 (lane / 32) + r of token wave * 32 + lane % 32);
// stored straight from there a store instruction writes 32-byte pieces 4 E
// bytes apart, the 128-byte lines reach the L2 in quarters and the 16.8 MB of
// logits of 65536 tokens x 64 experts cost 10 us.  Here the values go through
// LDS (stage: [128][E + 4] floats, any earlier use of it over) and leave as
// consecutive 16-byte pieces, whole lines per instruction (the 16.8 MB then
// cost 2 us).  rows: how many of the block's 128 tokens exist; out: their
// first row.  Ends with a barrier: the caller may reuse `stage` at once.
template <int NT, typename V>  // V: float[16] or a 16-float vector
__device__ __forceinline__ void store_logits_rows(const V (&v)[NT],
                                                  float* stage, int E,
                                                  float* __restrict__ out,
                                                  int rows) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ld = E + 4;
  float* row = stage + (wave * 32 + (lane & 31)) * ld;
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e0 = j * 32 + 8 * q + 4 * (lane >> 5);
      if (e0 < E)
        *reinterpret_cast<float4*>(row + e0) = make_float4(
            v[j][4 * q], v[j][4 * q + 1], v[j][4 * q + 2], v[j][4 * q + 3]);
    }
  __syncthreads();
  const int per_row = E >> 2;                    // 16-byte pieces per row
  for (int c = tid; c < rows * per_row; c += (int)blockDim.x) {
    const int r = c / per_row, piece = c - r * per_row;
    store_streaming(reinterpret_cast<uint4*>(out + (int64_t)r * E + piece * 4),
                    *reinterpret_cast<const uint4*>(stage + r * ld + piece * 4));
  }
  __syncthreads();
}

template <int NT>  // number of 32-expert tiles: E <= 32 * NT
__global__ __launch_bounds__(256) void router_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ wp,
    const float* __restrict__ bias, float* __restrict__ logits, int tokens,
    int M, int E) {
  constexpr int TOK = 128, BK = 64, ROWB = 128;
  constexpr int X_BYTES = TOK * ROWB, W_BYTES = NT * 32 * ROWB;
  constexpr int STAGE = X_BYTES + W_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char rl_smem[];
  const int b = blockIdx.y;
  const int t0 = blockIdx.x * TOK;
  const bf16_t* xb = x + (int64_t)b * tokens * M;
  const bf16_t* wb = wp + (int64_t)b * E * M;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // load instruction q covers tile rows 8q..8q+7; lane l fills slot
  // (row 8q + l/8, column l%8) and fetches chunk (l%8) ^ swizzle(row)
  int x_off[4], w_off[NT];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = (wave + 4 * j) * 8 + (lane >> 3);
    x_off[j] = min(t0 + row, tokens - 1) * M + (((lane & 7) ^ rl_swizzle(row)) * 8);
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int row = (wave + 4 * j) * 8 + (lane >> 3);
    w_off[j] = min(row, E - 1) * M + (((lane & 7) ^ rl_swizzle(row)) * 8);
  }
  // Block b walks the K tiles starting at tile b % nk and wraps around: the
  // blocks run in step, and with rows a power of two apart all of them asking
  // for the same 128-byte column of their rows at the same moment lands on
  // few memory channels (measured: 20 % slower).
  const int nk = M / BK;
  const int rot = (int)(blockIdx.x % (unsigned)nk);
  auto issue = [&](int kt, int slot) {
    unsigned char* sx = rl_smem + slot * STAGE;
    unsigned char* sw = sx + X_BYTES;
    int kq = kt + rot;
    if (kq >= nk) kq -= nk;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      __builtin_amdgcn_global_load_lds(
          (rl_glb_void_t*)(xb + kq * BK + x_off[j]),
          (rl_lds_void_t*)(sx + (wave + 4 * j) * 1024), 16, 0, RL_STREAMING);
#pragma unroll
    for (int j = 0; j < NT; ++j)
      __builtin_amdgcn_global_load_lds(
          (rl_glb_void_t*)(wb + kq * BK + w_off[j]),
          (rl_lds_void_t*)(sw + (wave + 4 * j) * 1024), 16, 0, 0);
  };

  rl_f32x16_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

  const int fr = lane & 31, fc = lane >> 5;
  int x_frag[4], w_frag[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    const int col = ((kk * 2 + fc) ^ rl_swizzle(fr)) * 16;
    x_frag[kk] = (wave * 32 + fr) * ROWB + col;
    w_frag[kk] = fr * ROWB + col;
  }
  // Three slots, two K tiles in flight: the loop is bound by the latency of
  // one round trip to HBM per K tile, so what it moves per second is the bytes
  // it keeps in flight.  vmcnt retires in issue order: leaving the newest
  // tile's 4 + NT loads outstanding means tile kt has landed.  Passing the
  // barrier of step kt also means every wavefront has finished reading slot
  // (kt - 1) % 3, which the loads of tile kt + 2 then overwrite.
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  int slot = 0;
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk)
      __builtin_amdgcn_s_waitcnt(0x0070 | (4 + NT));  // vmcnt(4+NT) lgkmcnt(0)
    else
      __builtin_amdgcn_s_waitcnt(0x0070);             // vmcnt(0) lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kt + 2 < nk) issue(kt + 2, slot == 0 ? 2 : slot - 1);
    const unsigned char* sx = rl_smem + slot * STAGE;
    slot = slot == 2 ? 0 : slot + 1;
    const unsigned char* sw = sx + X_BYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const rl_bf16x8_t xf = *reinterpret_cast<const rl_bf16x8_t*>(sx + x_frag[kk]);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const rl_bf16x8_t wf =
            *reinterpret_cast<const rl_bf16x8_t*>(sw + w_frag[kk] + j * 32 * ROWB);
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc[j], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // every wavefront is done with the ring: reuse it
  if (bias != nullptr) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        // E % 4 == 0, so the four experts are in range together
        const int e0 = min(j * 32 + 8 * q + 4 * (lane >> 5), E - 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[j][4 * q + r] += bias[e0 + r];
      }
  }
  store_logits_rows<NT>(acc, reinterpret_cast<float*>(rl_smem), E,
                        logits + ((int64_t)b * tokens + t0) * E,
                        min(TOK, tokens - t0));
}

// ---------------------------------------------------------------------------
// Gating step 1: per token softmax, top-2, gate normalisation, second-place
// policy; per block column sums of the balancing-loss proxies.
// Grid (blocks per group, G); one thread per token; the logits tile is staged
// in LDS with row stride E+1 so that per-thread row walks are conflict-free.
// ---------------------------------------------------------------------------
// Accesses that are coherent across the GPU's compute dies without a cache
// flush.  Each die (XCD) has its own L2; an ordinary store may sit there, and
// an ordinary load may hit a stale line there, until a device-scope fence
// writes back / invalidates that whole L2 -- too expensive to issue from
// every block of a kernel whose other blocks are still streaming through the
// same L2.  A relaxed atomic store / load at device scope is a write-through
// store / a load that bypasses lines the L2 cannot vouch for.  The blocks of
// the single-launch gating kernel exchange their data only through these:
// the writer waits until its stores have completed (vmcnt 0) before it bumps
// the arrival counter, the reader loads after it has seen the counter.
template <typename T>
__device__ __forceinline__ void st_dev(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ T ld_dev(const T* p) {
  return __hip_atomic_load(const_cast<T*>(p), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long pack_i2(int a, int b) {
  return (unsigned long long)(unsigned)a | ((unsigned long long)(unsigned)b << 32);
}
__device__ __forceinline__ unsigned long long pack_f2(float a, float b) {
  return pack_i2((int)__float_as_uint(a), (int)__float_as_uint(b));
}
// this wavefront's global stores (and loads) have completed
__device__ __forceinline__ void wait_stores() {
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0), nothing else
  asm volatile("" ::: "memory");
}

struct GateParams {
  int G, S, E, C;
  int policy;
  float threshold;      // float32(threshold)            (moe.py:1460)
  float inv_threshold;  // float32(1 / max(thr, 1e-9))   (moe.py:1465)
  int use_second_place_loss;
  int num_microbatches;
  int importance_from_slot_gate;  // importance = 0.5*((w>0.5)+(w>0))
  int tt;    // tokens per block of step 1
  int nblk;  // blocks per group of step 1
  int router;          // ROUTER_TOP2 or ROUTER_SWITCH
  int has_importance;  // switch loss: the proxy is masked per token
  int use_z_loss;      // switch: add z_loss_coef * z_loss (moe.py:1253-1266)
  float z_loss_coef;
  int rank_by_gate;    // switch_max: slots by descending gate (moe.py:1033-1039)
};

constexpr int ROUTER_TOP2 = 0;    // _top_2_gating, moe.py:1312-1513
constexpr int ROUTER_SWITCH = 1;  // _switch_gating, moe.py:1176-1309
constexpr int GSUM = 4;  // floats per group: loss term 1, term 2, #(imp==1), z
// Largest group every gating entry accepts (the reference's moe_group_size
// defaults to 1024, moe.py:139).  The capacity kernel keeps a group's expert
// ids in LDS (6 bytes per token) and the one-launch tail keeps slot prefixes
// in 16 bits: both rely on it.
constexpr int GATE_MAX_GROUP = 16384;

// bit 0 of the step-1 `kept` byte: the token competes for a slot (mask_k after
// importance and policy); bit 1 (second choice only): mask_2 before the policy,
// which is what the second-place loss counts (moe.py:1430).
//
// gate_select_tile does the work for `ntok` tokens (tokens t0 .. of group g,
// block `blk` of the group) whose logits already sit in LDS as tile[ntok][ld];
// every thread of the block must call it.
//
// With `ch` (LDS, 3 * ch_stride int16) the expert a token competes for with
// its first / second choice, and the expert the loss's extra count sees, also
// go there (-1 = none) for the in-block ranking of the single-launch kernel,
// which then writes `pos` itself.
template <typename IT>
__device__ __forceinline__ void gate_select_tile(
    float* tile, float* isone, int ld, int ntok, int g, int blk, int t0,
    const IT* __restrict__ importance, const float* __restrict__ second_uniform,
    const GateParams& p, int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    float* __restrict__ part1, float* __restrict__ part2,
    int16_t* ch = nullptr, int ch_stride = 0) {
  const int E = p.E, S = p.S;
  const int tid = threadIdx.x;
  float qscale = 0.f, zterm = 0.f;
  int i1 = 0;
  bool sel1 = false;
  if (tid < ntok) {
    float* row = tile + tid * ld;
    const int64_t t = (int64_t)g * S + t0 + tid;
    float m = row[0];
    for (int e = 1; e < E; ++e) m = fmaxf(m, row[e]);       // reduce_max
    const float negm = -m;
    float s = 0.f;
    for (int e = 0; e < E; ++e) s += expf(row[e] + negm);   // exp, reduce_sum
    const float neglse = -(logf(s) + m);                    // log + max
    float g1 = -1.f;
    for (int e = 0; e < E; ++e) {
      float pe = expf(row[e] + neglse);                     // exp(log_softmax)
      row[e] = pe;
      if (pe > g1) { g1 = pe; i1 = e; }                     // first argmax
    }
    sel1 = true;
    if (p.router == ROUTER_SWITCH && second_uniform != nullptr) {
      // policy "sample" (moe.py:1213-1216): the expert is the first arg-max of
      // the caller's choice logits [G,S,E] (router logits plus Gumbel noise
      // times the temperature, ops.py:5070-5086), which arrive through the
      // pointer the top-2 mode uses for its uniform samples; the gate is the
      // softmax probability of that expert (mtf.gather of raw_gates)
      const float* ch = second_uniform + t * E;
      float best = ch[0];
      i1 = 0;
      for (int e = 1; e < E; ++e) {
        const float v = ch[e];
        if (v > best) { best = v; i1 = e; }
      }
      g1 = row[i1];
    }
    if (p.router == ROUTER_SWITCH) {
      // one choice, raw probability as the gate (moe.py:1207-1228); the load
      // balancing loss counts every token's arg-max (density_1 is taken
      // before the importance mask, moe.py:1224) and an unmasked proxy
      if (importance != nullptr)
        sel1 = (load_f32<IT>(importance + t) == 1.0f);
      if (!sel1) g1 = g1 * 0.0f;
      idx[t * 2 + 0] = i1;
      idx[t * 2 + 1] = 0;
      if (ch == nullptr) {
        pos[t * 2 + 0] = 0;
        pos[t * 2 + 1] = 0;
      } else {
        ch[tid] = sel1 ? (int16_t)i1 : (int16_t)-1;
        ch[ch_stride + tid] = -1;
        ch[2 * ch_stride + tid] = (int16_t)i1;
      }
      gate[t * 2 + 0] = g1;
      gate[t * 2 + 1] = 0.0f;
      kept[t * 2 + 0] = (sel1 ? 1 : 0) | 2;   // bit 1: counted by density_1
      kept[t * 2 + 1] = 0;
      isone[tid] = 1.0f;
      const float lse = -neglse;                            // reduce_logsumexp
      zterm = sel1 ? lse * lse : 0.0f;                      // moe.py:1256-1259
    } else {
    bool sel2 = true;
    if (importance != nullptr) {
      float imp = load_f32<IT>(importance + t);
      if (p.importance_from_slot_gate)                      // moe.py:725-727
        imp = 0.5f * ((imp > 0.5f ? 1.0f : 0.0f) + (imp > 0.0f ? 1.0f : 0.0f));
      sel1 = (imp == 1.0f);                                 // moe.py:1402-1404
      sel2 = (imp > 0.0f);                                  // moe.py:1411
    }
    if (!sel1) g1 = g1 * 0.0f;
    // gates_without_top_1 = raw_gates * (1 - mask_1); its first argmax.
    float g2 = -1.f, qsum = 0.f;
    int i2 = 0;
    for (int e = 0; e < E; ++e) {
      float keep = (sel1 && e == i1) ? 0.0f : 1.0f;         // 1 + (-mask_1)
      float q = row[e] * keep;
      qsum += q;
      if (q > g2) { g2 = q; i2 = e; }
    }
    const float denom = (g1 + g2) + 1e-9f;                  // moe.py:1413
    const float r = 1.0f / denom;                           // reciprocal
    const float g1n = g1 * r, g2n = g2 * r;
    const bool sel2_loss = sel2;
    if (p.policy == MESH_MOE_SECOND_NONE) {
      sel2 = false;
    } else if (p.policy == MESH_MOE_SECOND_THRESHOLD) {
      sel2 = sel2 && (g2n > p.threshold);
    } else if (p.policy == MESH_MOE_SECOND_RANDOM) {
      sel2 = sel2 && (second_uniform[t] < g2n * p.inv_threshold);
    }
    idx[t * 2 + 0] = i1;
    idx[t * 2 + 1] = i2;
    if (ch == nullptr) {
      pos[t * 2 + 0] = 0;
      pos[t * 2 + 1] = 0;
    } else {
      ch[tid] = sel1 ? (int16_t)i1 : (int16_t)-1;
      ch[ch_stride + tid] = sel2 ? (int16_t)i2 : (int16_t)-1;
      ch[2 * ch_stride + tid] = sel2_loss ? (int16_t)i2 : (int16_t)-1;
    }
    gate[t * 2 + 0] = g1n;
    gate[t * 2 + 1] = g2n;
    kept[t * 2 + 0] = sel1 ? 1 : 0;
    kept[t * 2 + 1] = (sel2 ? 1 : 0) | (sel2_loss ? 2 : 0);
    isone[tid] = sel1 ? 1.0f : 0.0f;
    qscale = 1.0f / (qsum + 1e-9f);                         // moe.py:1433-1434
    }
  }
  __syncthreads();
  // density_1_proxy partial: sum over the block's tokens of p * (imp == 1)
  for (int e = tid; e < E; e += blockDim.x) {
    float s = 0.f;
    for (int r = 0; r < ntok; ++r) s += tile[r * ld + e] * isone[r];
    part1[((int64_t)g * p.nblk + blk) * E + e] = s;
  }
  if (p.router == ROUTER_SWITCH) {
    // per-block sums for the z-loss: column 0 = sum of logsumexp^2 over the
    // tokens with importance 1, column 1 = how many those are
    __syncthreads();
    if (tid < ntok) {
      tile[tid * ld + 0] = zterm;
      tile[tid * ld + 1] = sel1 ? 1.0f : 0.0f;
    }
    __syncthreads();
    if (tid < 2) {
      float s = 0.f;
      for (int r = 0; r < ntok; ++r) s += tile[r * ld + tid];
      part2[((int64_t)g * p.nblk + blk) * E + tid] = s;
    }
  } else if (p.use_second_place_loss) {
    __syncthreads();
    if (tid < ntok) {
      float* row = tile + tid * ld;
      for (int e = 0; e < E; ++e) {
        float keep = (sel1 && e == i1) ? 0.0f : 1.0f;
        row[e] = (row[e] * keep) * qscale;
      }
    }
    __syncthreads();
    for (int e = tid; e < E; e += blockDim.x) {
      float s = 0.f;
      for (int r = 0; r < ntok; ++r) s += tile[r * ld + e];
      part2[((int64_t)g * p.nblk + blk) * E + e] = s;
    }
  }
}

// ---------------------------------------------------------------------------
// gate_select_tile for the projection kernel, straight from the matrix-core
// accumulators: 256 threads, 128 tokens, two lanes per token.  After the
// 32x32x16 MFMAs lane l of a wavefront holds, for token l % 32 and per
// 32-expert tile j, the logits of experts 32 j + 8 q + 4 (l / 32) + r (q, r =
// 0..3): lanes l and l + 32 together hold the token's whole row, in alternating
// groups of four experts.  Each lane does the exponentials of its half (two per
// expert, the bulk of the work); every float32 sum still runs in expert order
// (the running sum changes lanes after every group of four) and a tie between
// the two lanes' arg-max candidates goes to the lower expert, so every
// per-token result is bit for bit that of gate_select_tile.  The probabilities
// go to LDS (tile [128][ld], ld % 4 == 0) for the per-block column sums of the
// loss, which are split over four row ranges; colpart: LDS [4][E] floats.
// ---------------------------------------------------------------------------
template <int NT, typename IT>
__device__ __forceinline__ void gate_select_acc_tile(
    const float (&xin)[NT][16], float* tile, float* isone, int ld, int g,
    int blk, int t0, const IT* __restrict__ importance,
    const float* __restrict__ second_uniform, const GateParams& p,
    int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    float* __restrict__ part1, float* __restrict__ part2, int16_t* ch,
    float* colpart) {
  constexpr int NTOK = 128;
  const int E = p.E, S = p.S;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5;
  const int tok = wave * 32 + (lane & 31);
  const bool sw = p.router == ROUTER_SWITCH;
  float* row = tile + tok * ld;
  const int64_t t = (int64_t)g * S + t0 + tok;
  // As the matrix cores leave them, register group (j, q) of the lower lane of
  // a token's pair holds experts 32 j + 8 q + 0..3 and the upper lane's
  // + 4..7: a sum in expert order changes lanes after every four experts.
  // With an even number of 32-expert blocks the pair first trades registers
  // (v_permlane32_swap: the upper half of one register against the lower half
  // of another), after which the lower lane holds the whole of block 2 jp in
  // its groups (2 jp, q), (2 jp + 1, q) -- experts 8 q + 0..3 and 8 q + 4..7 --
  // and the upper lane the whole of block 2 jp + 1: a sum in expert order then
  // changes lanes once per 32 experts.
  constexpr bool SWAPPED = NT % 2 == 0;
  float x[NT][16];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) x[j][i] = xin[j][i];
  if constexpr (SWAPPED) {
#pragma unroll
    for (int jp = 0; jp < NT / 2; ++jp)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const auto sw2 = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(x[2 * jp][i]), __float_as_uint(x[2 * jp + 1][i]),
            false, false);
        x[2 * jp][i] = __uint_as_float(sw2[0]);
        x[2 * jp + 1][i] = __uint_as_float(sw2[1]);
      }
  }
  // first expert of this lane's group (j, q); the group exists if it is < E
  auto first = [&](int j, int q) {
    return SWAPPED ? ((j & ~1) + half) * 32 + 8 * q + 4 * (j & 1)
                   : j * 32 + 8 * q + 4 * half;
  };
  // calls fn(j, q) for the lane's groups in ascending expert order
  auto for_groups = [&](auto fn) {
    if constexpr (SWAPPED) {
#pragma unroll
      for (int jp = 0; jp < NT / 2; ++jp)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          fn(2 * jp, q);
          fn(2 * jp + 1, q);
        }
    } else {
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) fn(j, q);
    }
  };
  // the partner's candidate wins if it is larger, or equal with a lower index
  auto take_other = [&](float mine, int mi, float other, int oi) {
    return other > mine || (other == mine && oi < mi);
  };
  // a float32 sum over the experts in index order: the lanes of a pair take
  // turns, the running value changing lanes when the next expert lives in the
  // other lane
  auto ordered_sum = [&](const float (&v)[NT][16]) {
    float s = 0.f;
    if constexpr (SWAPPED) {
#pragma unroll
      for (int jp = 0; jp < NT / 2; ++jp)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          if (half == hh) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
              for (int jj = 0; jj < 2; ++jj)
                if (first(2 * jp + jj, q) < E) {
#pragma unroll
                  for (int r = 0; r < 4; ++r) s += v[2 * jp + jj][4 * q + r];
                }
          }
          s = __shfl_xor(s, 32);
        }
    } else {
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bool mine = first(j, q) < E;
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) {
            if (half == hh && mine) {
#pragma unroll
              for (int r = 0; r < 4; ++r) s += v[j][4 * q + r];
            }
            s = __shfl_xor(s, 32);
          }
        }
    }
    return __shfl(s, lane & 31);      // the lower lane holds the final value
  };

  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (first(j, q) < E) {
#pragma unroll
        for (int r = 0; r < 4; ++r) m = fmaxf(m, x[j][4 * q + r]);   // reduce_max
      }
  m = fmaxf(m, __shfl_xor(m, 32));
  const float negm = -m;
  float pr[NT][16];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) pr[j][i] = expf(x[j][i] + negm);    // exp
  const float ssum = ordered_sum(pr);                                // reduce_sum
  const float neglse = -(logf(ssum) + m);                            // log + max
  float g1 = -1.f;
  int i1 = 0;
  for_groups([&](int j, int q) {
    if (first(j, q) < E) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float pe = expf(x[j][4 * q + r] + neglse);   // exp(log_softmax)
        pr[j][4 * q + r] = pe;
        if (pe > g1) { g1 = pe; i1 = first(j, q) + r; }    // first argmax
      }
      *reinterpret_cast<float4*>(row + first(j, q)) = make_float4(
          pr[j][4 * q], pr[j][4 * q + 1], pr[j][4 * q + 2], pr[j][4 * q + 3]);
    }
  });
  {
    const float og = __shfl_xor(g1, 32);
    const int oi = __shfl_xor(i1, 32);
    if (take_other(g1, i1, og, oi)) { g1 = og; i1 = oi; }
  }
  bool sel1 = true;
  if (sw && second_uniform != nullptr) {
    // policy "sample": first arg-max of the caller's choice logits
    const float* cl = second_uniform + t * E;
    float best = -INFINITY;
    int bi = E;
    for_groups([&](int j, int q) {
      if (first(j, q) < E) {
        const float4 c4 = *reinterpret_cast<const float4*>(cl + first(j, q));
        const float cv[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (bi == E || cv[r] > best) { best = cv[r]; bi = first(j, q) + r; }
      }
    });
    const float ob = __shfl_xor(best, 32);
    const int oi = __shfl_xor(bi, 32);
    if (take_other(best, bi, ob, oi)) bi = oi;
    i1 = bi;
    __syncthreads();           // the partner's half of the row is in LDS
    g1 = row[i1];
  }
  float qscale = 0.f, zterm = 0.f;
  if (sw) {
    if (importance != nullptr)
      sel1 = (load_f32<IT>(importance + t) == 1.0f);
    if (!sel1) g1 = g1 * 0.0f;
    if (half == 0) {
      st_dev(reinterpret_cast<unsigned long long*>(idx + t * 2), pack_i2(i1, 0));
      st_dev(reinterpret_cast<unsigned long long*>(gate + t * 2),
             pack_f2(g1, 0.0f));
    } else {
      st_dev(reinterpret_cast<uint16_t*>(kept + t * 2),
             (uint16_t)((sel1 ? 1 : 0) | 2));
      if (ch == nullptr) {
        *reinterpret_cast<int2*>(pos + t * 2) = make_int2(0, 0);
      } else {
        ch[tok] = sel1 ? (int16_t)i1 : (int16_t)-1;
        ch[NTOK + tok] = -1;
        ch[2 * NTOK + tok] = (int16_t)i1;
      }
      isone[tok] = 1.0f;
    }
    const float lse = -neglse;
    zterm = sel1 ? lse * lse : 0.0f;
  } else {
    bool sel2 = true;
    if (importance != nullptr) {
      float imp = load_f32<IT>(importance + t);
      if (p.importance_from_slot_gate)
        imp = 0.5f * ((imp > 0.5f ? 1.0f : 0.0f) + (imp > 0.0f ? 1.0f : 0.0f));
      sel1 = (imp == 1.0f);
      sel2 = (imp > 0.0f);
    }
    if (!sel1) g1 = g1 * 0.0f;
    // gates_without_top_1 = raw_gates * (1 - mask_1), in place; its first argmax
    float g2 = -1.f;
    int i2 = 0;
    for_groups([&](int j, int q) {
      if (first(j, q) < E) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int e = first(j, q) + r;
          const float keep = (sel1 && e == i1) ? 0.0f : 1.0f;
          const float qv = pr[j][4 * q + r] * keep;
          pr[j][4 * q + r] = qv;
          if (qv > g2) { g2 = qv; i2 = e; }
        }
      }
    });
    {
      const float og = __shfl_xor(g2, 32);
      const int oi = __shfl_xor(i2, 32);
      if (take_other(g2, i2, og, oi)) { g2 = og; i2 = oi; }
    }
    const float denom = (g1 + g2) + 1e-9f;
    const float r = 1.0f / denom;
    const float g1n = g1 * r, g2n = g2 * r;
    const bool sel2_loss = sel2;
    if (p.policy == MESH_MOE_SECOND_NONE) {
      sel2 = false;
    } else if (p.policy == MESH_MOE_SECOND_THRESHOLD) {
      sel2 = sel2 && (g2n > p.threshold);
    } else if (p.policy == MESH_MOE_SECOND_RANDOM) {
      sel2 = sel2 && (second_uniform[t] < g2n * p.inv_threshold);
    }
    if (half == 0) {
      st_dev(reinterpret_cast<unsigned long long*>(idx + t * 2), pack_i2(i1, i2));
      st_dev(reinterpret_cast<unsigned long long*>(gate + t * 2),
             pack_f2(g1n, g2n));
    } else {
      st_dev(reinterpret_cast<uint16_t*>(kept + t * 2), (uint16_t)(
          (sel1 ? 1 : 0) | ((sel2 ? 1 : 0) | (sel2_loss ? 2 : 0)) << 8));
      if (ch == nullptr) {
        *reinterpret_cast<int2*>(pos + t * 2) = make_int2(0, 0);
      } else {
        ch[tok] = sel1 ? (int16_t)i1 : (int16_t)-1;
        ch[NTOK + tok] = sel2 ? (int16_t)i2 : (int16_t)-1;
        ch[2 * NTOK + tok] = sel2_loss ? (int16_t)i2 : (int16_t)-1;
      }
      isone[tok] = sel1 ? 1.0f : 0.0f;
    }
    if (p.use_second_place_loss)
      qscale = 1.0f / (ordered_sum(pr) + 1e-9f);            // moe.py:1433-1434
  }
  __syncthreads();
  // column sums over the block's tokens, four row ranges per column
  auto column_sums = [&](int ncol, bool weighted, float* out) {
    for (int i = tid; i < 4 * ncol; i += blockDim.x) {
      const int e = i % ncol, q4 = i / ncol;
      float acc = 0.f;
      // (the reads of a batch fly together; the additions keep their order)
      const float* col = tile + q4 * (NTOK / 4) * ld + e;
      const float* one = isone + q4 * (NTOK / 4);
#pragma unroll 8
      for (int r = 0; r < NTOK / 4; ++r)
        acc += weighted ? col[r * ld] * one[r] : col[r * ld];
      colpart[q4 * ncol + e] = acc;
    }
    __syncthreads();
    for (int e = tid; e < ncol; e += blockDim.x)
      st_dev(out + ((int64_t)g * p.nblk + blk) * E + e,
             ((colpart[e] + colpart[ncol + e]) + colpart[2 * ncol + e]) +
                 colpart[3 * ncol + e]);
  };
  column_sums(E, true, part1);       // density_1_proxy: p * (imp == 1)
  if (sw) {
    // z-loss: column 0 = sum of logsumexp^2 over the tokens of importance 1,
    // column 1 = how many those are
    __syncthreads();
    if (half == 0) {
      row[0] = zterm;
      row[1] = sel1 ? 1.0f : 0.0f;
    }
    __syncthreads();
    column_sums(2, false, part2);
  } else if (p.use_second_place_loss) {
    // the proxy of the second-place loss: (gates without the first) / their sum
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (first(j, q) < E)
          *reinterpret_cast<float4*>(row + first(j, q)) = make_float4(
              pr[j][4 * q] * qscale, pr[j][4 * q + 1] * qscale,
              pr[j][4 * q + 2] * qscale, pr[j][4 * q + 3] * qscale);
    __syncthreads();
    column_sums(E, false, part2);
  }
}

template <typename IT>
__global__ __launch_bounds__(256) void gate_select_kernel(
    const float* __restrict__ logits, const IT* __restrict__ importance,
    const float* __restrict__ second_uniform, GateParams p,
    int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    float* __restrict__ part1, float* __restrict__ part2) {
  extern __shared__ float smem[];
  const int E = p.E, S = p.S;
  const int ld = E + 1;
  float* tile = smem;                                  // [tt][E+1]
  float* isone = smem + (size_t)p.tt * ld;             // [tt]
  const int g = blockIdx.y;
  const int blk = blockIdx.x;
  const int t0 = blk * p.tt;
  const int ntok = min(p.tt, S - t0);
  const int tid = threadIdx.x;
  const float* src = logits + ((int64_t)g * S + t0) * E;
  for (int i = tid; i < ntok * E; i += blockDim.x) {
    int r = i / E, c = i - r * E;
    tile[r * ld + c] = src[i];
  }
  __syncthreads();
  gate_select_tile<IT>(tile, isone, ld, ntok, g, blk, t0, importance,
                       second_uniform, p, idx, pos, gate, kept, part1, part2);
}

// ---------------------------------------------------------------------------
// Capacity positions and the loss inside the projection kernel's launch.
//
// Every block ranks the choices of its own 128 tokens (gate_rank_tile: per
// expert a wavefront ballot over 64 tokens and the number of set bits below
// the lane, then the count of the block's other half) and publishes its
// per-expert counts.  The block of a group that arrives last at the group's
// counter (gate_group_tail) turns the counts into each block's first slot per
// expert, finishes every token of the group (slot = first slot of its block +
// rank in the block; second choices behind the kept first choices), writes
// `fill` and the group's loss term; the group that finishes last adds the
// terms up.  Nobody waits for anybody, so the scheme does not depend on which
// blocks are resident together.
//
// A counter is a 64-bit word: call number << 16 | arrivals.  A word that does
// not carry the current call's number counts as zero, so the workspace may
// hold anything when the call starts; the last arrival leaves zero behind.
// ---------------------------------------------------------------------------
struct GateParams;
template <bool COHERENT>
__device__ __forceinline__ void gate_loss_value(const GateParams& p,
                                                const float* gsum, float* loss);

struct FusedTail {
  int32_t* bcnt;              // [G][nblk][3][E] per-block counts
  unsigned long long* gctr;   // [G] arrivals per group
  unsigned long long* fctr;   // [1] groups done
  float* gsum;                // [G][GSUM]
  int32_t* fill;              // [G][E]
  float* loss;                // [1]
  unsigned long long call;    // number of this call, < 2^48, never 0
};

// Puts a counter word into this call's state "no arrivals yet" if it holds
// zero, which is what the last arrival of the previous use leaves behind.
// Nobody waits for the result: a word that held something else (a workspace
// used for the first time) is handled by the arrivals themselves.
__device__ __forceinline__ void counter_prepare(unsigned long long* word,
                                                unsigned long long call) {
  unsigned long long zero = 0ull;
  (void)__hip_atomic_compare_exchange_strong(
      word, &zero, call << 16, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
      __HIP_MEMORY_SCOPE_AGENT);
}

// true for the last of `expected` arrivals; one thread per arrival.  The
// common case is one fetch-add on a word that counter_prepare stamped long
// ago.  An arrival that finds another stamp (its add then changed a word
// nobody relies on) installs the stamp itself or, if somebody else just did,
// adds again: every arrival ends with exactly one successful operation on a
// word that carries this call's stamp.
__device__ __forceinline__ bool arrive_is_last(unsigned long long* word,
                                               unsigned long long call,
                                               unsigned expected) {
  unsigned long long old = __hip_atomic_fetch_add(
      word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if ((old >> 16) == call) return (unsigned)((old + 1) & 0xffffu) == expected;
  old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (;;) {
    if ((old >> 16) == call) {
      old = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
      return (unsigned)((old + 1) & 0xffffu) == expected;
    }
    const unsigned long long seen = atomicCAS(word, old, (call << 16) | 1ull);
    if (seen == old) return expected == 1u;
    old = seen;
  }
}

// Ranks of the block's choices.  ch [3][128] int16 in LDS as written by
// gate_select_tile; wcnt [3][2][E] int32 in LDS.  Wavefront w ranks choice
// w / 2 of tokens 64 (w % 2) ..; with `loss2` wavefronts 0 and 1 also count
// the third array.  A lane's rank is the number of lower lanes of its
// wavefront that name the same expert.  Writes pos (rank within the block)
// for competing choices, 0 otherwise, and the block's counts to
// bcnt_blk [3][E].
__device__ __forceinline__ void gate_rank_tile(
    const int16_t* ch, int32_t* wcnt, int E, bool loss2, int64_t tok0,
    int32_t* __restrict__ pos, int32_t* __restrict__ bcnt_blk) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = wave >> 1, half = wave & 1;
  // bits an expert id has
  const int nbits = 32 - __builtin_clz((unsigned)max(E - 1, 1));
  // The lanes of this wavefront that name the same expert as this lane, from
  // one ballot per bit of the id (instead of one per expert): a lane keeps the
  // lanes whose bit equals its own.  id < 0: not competing, matches nobody.
  auto same_choice = [&](int id) {
    unsigned long long match = __ballot(id >= 0);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = ((id >> b) & 1) != 0;
      const unsigned long long mb = __ballot(bit);
      match &= bit ? mb : ~mb;
    }
    return id >= 0 ? match : 0ull;
  };
  const unsigned long long before =
      lane == 0 ? 0ull : (~0ull >> (64 - lane));      // the lanes below this one
  auto clear_counts = [&](int32_t* dst) {
    for (int e = lane; e < E; e += 64) dst[e] = 0;
  };
  const int mine = ch[c * 128 + half * 64 + lane];
  int32_t* my_cnt = wcnt + (c * 2 + half) * E;
  clear_counts(my_cnt);
  const unsigned long long match = same_choice(mine);
  int rank = (int)__popcll(match & before);
  // the first lane of every expert's choosers writes the expert's count (LDS
  // keeps a wavefront's writes in program order: after the clearing)
  if (mine >= 0 && rank == 0) my_cnt[mine] = (int)__popcll(match);
  if (loss2 && c == 0) {
    const int third = ch[2 * 128 + half * 64 + lane];
    int32_t* cnt3 = wcnt + (4 + half) * E;
    clear_counts(cnt3);
    const unsigned long long m3 = same_choice(third);
    if (third >= 0 && (m3 & before) == 0ull) cnt3[third] = (int)__popcll(m3);
  }
  __syncthreads();
  if (half == 1 && mine >= 0) rank += wcnt[(c * 2) * E + mine];
  st_dev(pos + (tok0 + half * 64 + lane) * 2 + c, mine >= 0 ? rank : 0);
  for (int i = tid; i < 3 * E; i += blockDim.x) {
    const int cc = i / E, e = i - cc * E;
    st_dev(bcnt_blk + i, (cc < 2 || loss2) ? wcnt[(cc * 2) * E + e] +
                                                 wcnt[(cc * 2 + 1) * E + e]
                                           : 0);
  }
}

// What the last block of group g does (all 256 threads; smem is the block's
// whole dynamic LDS, free by now).  Same results, bit for bit, as
// gate_capacity_kernel + gate_loss_kernel for slots in token order.
__device__ __forceinline__ void gate_group_tail(
    unsigned char* smem, const GateParams& p, const FusedTail& ft, int g,
    const int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    const float* __restrict__ part1, const float* __restrict__ part2) {
  const int S = p.S, E = p.E, C = p.C, nblk = p.nblk;
  const int tid = threadIdx.x;
  const bool sw = p.router == ROUTER_SWITCH;
  const bool loss2 = p.use_second_place_loss != 0 || sw;
  // First slots per block and expert.  16 bits suffice: a prefix is at most
  // the number of tokens of the earlier blocks, below S <= GATE_MAX_GROUP
  // (every gating entry refuses larger groups).
  static_assert(GATE_MAX_GROUP <= 65535, "the block prefixes are 16 bits wide");
  uint16_t* pre1 = reinterpret_cast<uint16_t*>(smem);          // [nblk][E]
  uint16_t* pre2 = pre1 + (size_t)nblk * E;                    // [nblk][E]
  int32_t* tot = reinterpret_cast<int32_t*>(
      smem + (((size_t)nblk * E * 4 + 15) & ~(size_t)15));     // [3][E]
  float* prod = reinterpret_cast<float*>(tot + 3 * E);         // [2][E]
  float* misc = prod + 2 * E;                                  // [4]
  int* last_group = reinterpret_cast<int*>(misc + 4);          // [1] (+ 3 pad)
  const int32_t* bc = ft.bcnt + (int64_t)g * nblk * 3 * E;
  const int64_t base = (int64_t)g * S;
  // Everything here comes from other compute units' stores, i.e. from memory,
  // one round trip per dependent access: the loads of the three parts (token
  // records, partial sums of the loss, per-block counts) are issued together
  // before anything is used.
  constexpr int U = 8;     // tokens per thread and trip
  constexpr int PB = 16;   // blocks whose partial sums are fetched up front
  int2 ex[U], rk[U];
  float2 gt[U];
  uint16_t kk[U];
  auto load_records = [&](int s0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * (int)blockDim.x;
      if (s < S) {
        const int64_t t = base + s;
        const unsigned long long e2 =
            ld_dev(reinterpret_cast<const unsigned long long*>(idx + t * 2));
        const unsigned long long r2 =
            ld_dev(reinterpret_cast<const unsigned long long*>(pos + t * 2));
        const unsigned long long g2 =
            ld_dev(reinterpret_cast<const unsigned long long*>(gate + t * 2));
        kk[u] = ld_dev(reinterpret_cast<const uint16_t*>(kept + t * 2));
        ex[u] = make_int2((int)(unsigned)e2, (int)(e2 >> 32));
        rk[u] = make_int2((int)(unsigned)r2, (int)(r2 >> 32));
        gt[u] = make_float2(__uint_as_float((unsigned)g2),
                            __uint_as_float((unsigned)(g2 >> 32)));
      }
    }
  };
  // Loads return in the order they were issued: the per-block counts, which
  // the prefixes below need first, go out before the (many more) record loads.
  auto load_counts = [&](int i, int (&cv)[PB]) {
    const int c = i / E, e = i - c * E;
#pragma unroll
    for (int b = 0; b < PB; ++b)
      cv[b] = (i < 3 * E && b < nblk && (c < 2 || loss2))
                  ? ld_dev(bc + ((int64_t)b * 3 + c) * E + e) : 0;
  };
  int cv0[PB];
  load_counts(tid, cv0);
  // thread e < E sums column e of part1, threads E .. 2E-1 column e of part2
  // (second-place loss: E columns; switch: columns 0 and 1), in block order
  const int pcol = tid < E ? tid : tid - E;
  const bool sums1 = tid < E;
  const bool sums2 = !sums1 && tid < 2 * E && loss2 && (!sw || pcol < 2);
  const float* pcolumn = (sums1 ? part1 : part2) + (int64_t)g * nblk * E + pcol;
  float pv[PB];
  if (sums1 || sums2) {
#pragma unroll
    for (int b = 0; b < PB; ++b)
      pv[b] = b < nblk ? ld_dev(pcolumn + (int64_t)b * E) : 0.f;
  }
  load_records(tid);
  // first slot of every block per expert: exclusive prefix over the blocks
  for (int i = tid; i < 3 * E; i += blockDim.x) {
    const int c = i / E, e = i - c * E;
    if (c == 2 && !loss2) { tot[i] = 0; continue; }
    uint16_t* pre = c == 0 ? pre1 : pre2;
    int cv[PB];
    if (i == tid) {
#pragma unroll
      for (int b = 0; b < PB; ++b) cv[b] = cv0[b];
    } else {
      load_counts(i, cv);
    }
    int run = 0;
#pragma unroll
    for (int b = 0; b < PB; ++b) {
      if (b < nblk) {
        if (c < 2) pre[b * E + e] = (uint16_t)run;
        run += cv[b];
      }
    }
    for (int b = PB; b < nblk; ++b) {
      const int v = ld_dev(bc + ((int64_t)b * 3 + c) * E + e);
      if (c < 2) pre[b * E + e] = (uint16_t)run;
      run += v;
    }
    tot[i] = run;
  }
  float psum = 0.f;
  if (sums1 || sums2) {
#pragma unroll
    for (int b = 0; b < PB; ++b)
      if (b < nblk) psum += pv[b];
    for (int b = PB; b < nblk; ++b) psum += ld_dev(pcolumn + (int64_t)b * E);
  }
  __syncthreads();
  // Per-expert outputs and the group's share of the balancing loss come first:
  // the group's arrival at the call's counter then travels while the records
  // are rewritten.
  if (sums2) {
    if (sw) misc[pcol] = psum;
    else prod[E + pcol] = psum;      // proxy of the second-place loss, for now
  }
  __syncthreads();
  if (tid < E) {
    const int t1 = tot[tid], t2 = tot[E + tid];
    const int k1 = min(t1, C);
    ft.fill[(int64_t)g * E + tid] = k1 + min(t2, C - k1);
    const float inv_s = (float)(1.0 / (double)S);
    const int dens = sw ? tot[2 * E + tid] : t1;
    prod[tid] = (psum * inv_s) * ((float)dens * inv_s);
    if (loss2 && !sw)
      prod[E + tid] = (prod[E + tid] * inv_s) * ((float)tot[2 * E + tid] * inv_s);
  }
  __syncthreads();
  if (tid == 0) {
    float s1 = 0.f, s2 = 0.f;
    for (int k = 0; k < E; ++k) s1 += prod[k];
    if (loss2 && !sw)
      for (int k = 0; k < E; ++k) s2 += prod[E + k];
    float* gs = ft.gsum + (int64_t)g * GSUM;
    st_dev(gs + 0, s1);
    st_dev(gs + 1, s2);
    st_dev(gs + 2, sw ? (E > 1 ? misc[1] : 0.f) : 0.f);
    st_dev(gs + 3, sw ? misc[0] : 0.f);
    st_dev(ft.gctr + g, 0ull);
    wait_stores();
    const bool last = arrive_is_last(ft.fctr, ft.call, (unsigned)p.G);
    if (last) st_dev(ft.fctr, 0ull);
    *last_group = last ? 1 : 0;
  }
  for (int s0 = tid; s0 < S; s0 += (int)blockDim.x * U) {
    if (s0 != tid) load_records(s0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * (int)blockDim.x;
      if (s >= S) continue;
      const int blk = s >> 7;
      uint16_t kout = 0;
      if (kk[u] & 1) {
        const int slot = pre1[blk * E + ex[u].x] + rk[u].x;
        rk[u].x = slot;
        if (slot < C) kout |= 1; else gt[u].x = gt[u].x * 0.0f;
      } else {
        rk[u].x = 0;
        gt[u].x = gt[u].x * 0.0f;
      }
      if (kk[u] & 0x100) {
        const int slot = min(tot[ex[u].y], C) + pre2[blk * E + ex[u].y] + rk[u].y;
        rk[u].y = slot;
        if (slot < C) kout |= 0x100; else gt[u].y = gt[u].y * 0.0f;
      } else {
        rk[u].y = 0;
        gt[u].y = gt[u].y * 0.0f;
      }
      kk[u] = kout;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * (int)blockDim.x;
      if (s < S) {
        const int64_t t = base + s;
        *reinterpret_cast<int2*>(pos + t * 2) = rk[u];
        *reinterpret_cast<uint16_t*>(kept + t * 2) = kk[u];
        *reinterpret_cast<float2*>(gate + t * 2) = gt[u];
      }
    }
  }
  // The last group to finish turns the groups' terms into the loss: all
  // threads fetch them (one round trip instead of one per group), one thread
  // adds them in group order.
  __syncthreads();
  const bool finishes_call = *last_group != 0;
  __syncthreads();                 // (the staging below overwrites the flag)
  if (finishes_call) {
    float* stage = reinterpret_cast<float*>(smem);     // the prefixes are done with
    const int n = p.G * GSUM;
    if (n <= 8192) {
      for (int i = tid; i < n; i += (int)blockDim.x) stage[i] = ld_dev(ft.gsum + i);
      __syncthreads();
      if (tid == 0) gate_loss_value<false>(p, stage, ft.loss);
    } else if (tid == 0) {
      gate_loss_value<true>(p, ft.gsum, ft.loss);
    }
  }
}

// ---------------------------------------------------------------------------
// Router projection fused with gating step 1: the K loop of router_mfma_kernel,
// then the block's 128 x E logits go from the accumulators to LDS (never to
// HBM unless `logits` is given) and gate_select_tile runs on them.  Needs the
// group size to be a multiple of 128 so that a block's tokens share a group.
// ---------------------------------------------------------------------------
template <int NT, typename IT>
__global__ __launch_bounds__(256) void router_gate_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ wp,
    const float* __restrict__ bias, float* __restrict__ logits,
    int64_t tokens_total, int M, const IT* __restrict__ importance,
    const float* __restrict__ second_uniform, GateParams p,
    int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    float* __restrict__ part1, float* __restrict__ part2,
    int tokens_per_batch, FusedTail ft) {
  constexpr int TOK = 128, BK = 64, ROWB = 128;
  constexpr int X_BYTES = TOK * ROWB, W_BYTES = NT * 32 * ROWB;
  constexpr int STAGE = X_BYTES + W_BYTES;
  extern __shared__ __attribute__((aligned(16))) unsigned char rl_smem[];
  __shared__ int last_of_group;
  const int E = p.E;
  const int64_t tok0 = (int64_t)blockIdx.x * TOK;       // first token, flat
  if (ft.bcnt != nullptr && threadIdx.x == 0) {
    // the first block of a group stamps the group's counter for this call
    if (tok0 % p.S == 0) counter_prepare(ft.gctr + tok0 / p.S, ft.call);
    if (blockIdx.x == 0) counter_prepare(ft.fctr, ft.call);
  }
  const int b = (int)(tok0 / tokens_per_batch);         // router weight set
  const bf16_t* xb = x + tok0 * M;
  const bf16_t* wb = wp + (int64_t)b * E * M;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  int x_off[4], w_off[NT];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = (wave + 4 * j) * 8 + (lane >> 3);
    x_off[j] = row * M + (((lane & 7) ^ rl_swizzle(row)) * 8);
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int row = (wave + 4 * j) * 8 + (lane >> 3);
    w_off[j] = min(row, E - 1) * M + (((lane & 7) ^ rl_swizzle(row)) * 8);
  }
  // Block b walks the K tiles starting at tile b % nk and wraps around: the
  // blocks run in step, and with rows a power of two apart all of them asking
  // for the same 128-byte column of their rows at the same moment lands on
  // few memory channels (measured: 20 % slower).
  const int nk = M / BK;
  const int rot = (int)(blockIdx.x % (unsigned)nk);
  auto issue = [&](int kt, int slot) {
    unsigned char* sx = rl_smem + slot * STAGE;
    unsigned char* sw = sx + X_BYTES;
    int kq = kt + rot;
    if (kq >= nk) kq -= nk;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      __builtin_amdgcn_global_load_lds(
          (rl_glb_void_t*)(xb + kq * BK + x_off[j]),
          (rl_lds_void_t*)(sx + (wave + 4 * j) * 1024), 16, 0, RL_STREAMING);
#pragma unroll
    for (int j = 0; j < NT; ++j)
      __builtin_amdgcn_global_load_lds(
          (rl_glb_void_t*)(wb + kq * BK + w_off[j]),
          (rl_lds_void_t*)(sw + (wave + 4 * j) * 1024), 16, 0, 0);
  };
  rl_f32x16_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  const int fr = lane & 31, fc = lane >> 5;
  int x_frag[4], w_frag[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    const int col = ((kk * 2 + fc) ^ rl_swizzle(fr)) * 16;
    x_frag[kk] = (wave * 32 + fr) * ROWB + col;
    w_frag[kk] = fr * ROWB + col;
  }
  // Three slots, two K tiles in flight: the loop is bound by the latency of
  // one round trip to HBM per K tile, so what it moves per second is the bytes
  // it keeps in flight.  vmcnt retires in issue order: leaving the newest
  // tile's 4 + NT loads outstanding means tile kt has landed.  Passing the
  // barrier of step kt also means every wavefront has finished reading slot
  // (kt - 1) % 3, which the loads of tile kt + 2 then overwrite.
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  int slot = 0;
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk)
      __builtin_amdgcn_s_waitcnt(0x0070 | (4 + NT));  // vmcnt(4+NT) lgkmcnt(0)
    else
      __builtin_amdgcn_s_waitcnt(0x0070);             // vmcnt(0) lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (kt + 2 < nk) issue(kt + 2, slot == 0 ? 2 : slot - 1);
    const unsigned char* sx = rl_smem + slot * STAGE;
    slot = slot == 2 ? 0 : slot + 1;
    const unsigned char* sw = sx + X_BYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const rl_bf16x8_t xf = *reinterpret_cast<const rl_bf16x8_t*>(sx + x_frag[kk]);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const rl_bf16x8_t wf =
            *reinterpret_cast<const rl_bf16x8_t*>(sw + w_frag[kk] + j * 32 * ROWB);
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc[j], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // every wavefront is done with the ring: reuse it

  // this lane's logits (+ bias), written out if the caller wants them
  float* tile = reinterpret_cast<float*>(rl_smem);
  const int ld = E + 4;
  float* isone = tile + TOK * ld;
  float xl[NT][16];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e0 = j * 32 + 8 * q + 4 * (lane >> 5);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[j][4 * q + r];
        if (e0 < E) {
          if (bias != nullptr) v += bias[e0 + r];
        } else {
          v = -INFINITY;     // not an expert: exp() = 0, never the maximum
        }
        xl[j][4 * q + r] = v;
      }
    }
  }
  if (logits != nullptr)
    store_logits_rows<NT>(xl, tile, E, logits + tok0 * E, TOK);
  const int g = (int)(tok0 / p.S);
  const int t0 = (int)(tok0 - (int64_t)g * p.S);
  int16_t* ch = reinterpret_cast<int16_t*>(isone + TOK);      // [3][TOK]
  int32_t* wcnt = reinterpret_cast<int32_t*>(ch + 3 * TOK);   // [3][2][E]
  float* colpart = reinterpret_cast<float*>(wcnt + 6 * E);    // [4][E]
  const int blk = t0 / TOK;
  // (one call for both uses: the selection is 64 exponentials per lane long,
  // and a second inlined copy is code the instruction cache has to fetch)
  gate_select_acc_tile<NT, IT>(
      xl, tile, isone, ld, g, blk, t0, importance, second_uniform, p, idx, pos,
      gate, kept, part1, part2, ft.bcnt == nullptr ? nullptr : ch, colpart);
  // without the tail's workspace, capacity positions and loss follow as
  // launches of their own
  if (ft.bcnt == nullptr) return;
  const bool loss2 = p.use_second_place_loss != 0 || p.router == ROUTER_SWITCH;
  gate_rank_tile(ch, wcnt, E, loss2, tok0, pos,
                 ft.bcnt + ((int64_t)g * p.nblk + blk) * 3 * E);
  // This block's records, counts and partial sums are out (write-through
  // stores, see st_dev): once every wavefront's stores have completed, one
  // thread arrives at the group's counter; the last block to arrive finishes
  // the group.
  wait_stores();
  __syncthreads();
  if (tid == 0)
    last_of_group =
        arrive_is_last(ft.gctr + g, ft.call, (unsigned)p.nblk) ? 1 : 0;
  __syncthreads();
  if (!last_of_group) return;
  gate_group_tail(rl_smem, p, ft, g, idx, pos, gate, kept, part1, part2);
  (void)tokens_total;
}

// ---------------------------------------------------------------------------
// Gating step 2: capacity positions for one group per block (moe.py:1472-1496).
// Thread (e = tid % EL, chunk = tid / EL) counts, over its chunk of the
// group's tokens, those whose choice is expert e; an exclusive prefix over the
// chunks gives the slot of each chunk's first chooser of e.  Then one thread
// per token adds the number of earlier choosers of its expert inside its own
// chunk: every lane runs the same short loop, where a walk per (expert, chunk)
// would have each wave step through every token of the chunk.  Second choices
// start after the kept first choices of the same expert.  The token's expert
// ids live in LDS as int16 (-1 = not competing).
// ---------------------------------------------------------------------------
constexpr int CAP_THREADS = 1024;

// How many of the eight int16 expert ids in v equal e (0 <= e < 1024; an id of
// -1, "not competing", never does).
__device__ __forceinline__ int cap_match8(const uint4& v, int e) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  const uint32_t ue = (uint32_t)e;
  int n = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    n += ((w[j] & 0xffffu) == ue ? 1 : 0) + ((w[j] >> 16) == ue ? 1 : 0);
  return n;
}

// Number of entries of ch[s_begin, s_end) equal to e; with `vec` the range
// starts 16-byte aligned and is read eight ids at a time.
__device__ __forceinline__ int cap_count(const int16_t* ch, int s_begin,
                                         int s_end, int e, bool vec) {
  int c = 0, s = s_begin;
  if (vec)
    for (; s + 8 <= s_end; s += 8)
      c += cap_match8(*reinterpret_cast<const uint4*>(ch + s), e);
  for (; s < s_end; ++s) c += (ch[s] == e);
  return c;
}

__global__ __launch_bounds__(CAP_THREADS) void gate_capacity_kernel(
    GateParams p, const int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    int32_t* __restrict__ fill, const float* __restrict__ part1,
    const float* __restrict__ part2, float* __restrict__ gsum, int el) {
  extern __shared__ __attribute__((aligned(16))) int32_t smem_i[];
  const int S = p.S, E = p.E, C = p.C;
  int32_t* cnt = smem_i;                        // [nchunks][el] = CAP_THREADS
  int32_t* pre = cnt + CAP_THREADS;             // [nchunks][el]: first slots
  int32_t* tot = pre + CAP_THREADS;             // [3][el]: total1,total2,loss2
  float* prod = reinterpret_cast<float*>(tot + 3 * el);  // [2][el]
  int16_t* c1 = reinterpret_cast<int16_t*>(prod + 2 * el);  // [S]
  int16_t* c2 = c1 + S;                                      // [S]
  int16_t* c2l = c2 + S;                                     // [S] (loss only)
  // first-choice gates of the group, for the by-gate slot order; float-aligned
  // because 3 * S int16 may end on an odd 2-byte boundary
  float* gl = reinterpret_cast<float*>(c2l + S + (S & 1));    // [S]
  // by-gate order only: the first-choice gates listed per expert (token order
  // within an expert), every token's place in that list, the experts' first
  // places
  float* lg = gl + S;                                         // [S]
  int32_t* lpos = reinterpret_cast<int32_t*>(lg + S);         // [S]
  int32_t* ebase = lpos + S;                                  // [el]
  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)g * S;
  const bool sw = p.router == ROUTER_SWITCH;
  // a third count per expert: the second-place loss's mask_2 before the
  // policy (top-2), or every token's arg-max for density_1 (switch)
  const bool loss2 = p.use_second_place_loss != 0 || sw;
  for (int s = tid; s < S; s += CAP_THREADS) {
    int64_t t = base + s;
    int a = idx[t * 2], b = idx[t * 2 + 1];
    uint8_t k1 = kept[t * 2], k2 = kept[t * 2 + 1];
    c1[s] = (k1 & 1) ? (int16_t)a : (int16_t)-1;
    c2[s] = (k2 & 1) ? (int16_t)b : (int16_t)-1;
    if (sw) c2l[s] = (k1 & 2) ? (int16_t)a : (int16_t)-1;
    else if (loss2) c2l[s] = (k2 & 2) ? (int16_t)b : (int16_t)-1;
    if (p.rank_by_gate) gl[s] = gate[t * 2];
  }
  __syncthreads();
  const int e = tid % el;
  const int chunk = tid / el;
  const int nchunks = CAP_THREADS / el;
  const int clen = (S + nchunks - 1) / nchunks;
  const int s_begin = min(S, chunk * clen);
  const int s_end = min(S, s_begin + clen);
  // 16-byte reads of the id arrays: c1 starts 8192 + 20 * el bytes into LDS,
  // c2 and c2l S and 2 S ids later, a chunk clen ids after the previous one
  const bool vec = (el % 4 == 0) && (S % 8 == 0) && (clen % 8 == 0);

  int count1 = 0;  // kept first choices of expert e (valid after choice 0)
  for (int choice = 0; choice < 2; ++choice) {
    const int16_t* ch = choice == 0 ? c1 : c2;
    cnt[chunk * el + e] = cap_count(ch, s_begin, s_end, e, vec);
    __syncthreads();
    int before = 0, total = 0;
    for (int k = 0; k < nchunks; ++k) {
      int v = cnt[k * el + e];
      total += v;
      if (k < chunk) before += v;
    }
    pre[chunk * el + e] = before + (choice == 0 ? 0 : count1);
    if (chunk == 0 && e < E) tot[choice * el + e] = total;
    if (choice == 0) count1 = min(total, C);
    __syncthreads();
    const bool by_gate = p.rank_by_gate && choice == 0;
    if (by_gate) {
      if (tid == 0) {
        int run = 0;
        for (int k = 0; k < E; ++k) { ebase[k] = run; run += tot[k]; }
      }
      __syncthreads();
    }
    for (int s = tid; s < S; s += CAP_THREADS) {
      const int ex = ch[s];
      if (ex < 0) continue;
      const int ck = s / clen;
      const int slot = pre[ck * el + ex] + cap_count(ch, ck * clen, s, ex, vec);
      if (by_gate) {
        // not the slot yet: the token's place among its expert's choosers
        lpos[s] = ebase[ex] + slot;
        lg[ebase[ex] + slot] = gl[s];
        continue;
      }
      const int64_t t = base + s;
      const bool ok = slot < C;
      pos[t * 2 + choice] = slot;
      kept[t * 2 + choice] = ok ? 1 : 0;
      if (!ok) gate[t * 2 + choice] = gate[t * 2 + choice] * 0.0f;
    }
    __syncthreads();
  }
  if (p.rank_by_gate) {
    // switch_max: expert e keeps its C choosers with the largest gate; slot =
    // rank by (gate descending, token ascending), the order of tf.math.top_k
    for (int s = tid; s < S; s += CAP_THREADS) {
      const int ex = c1[s];
      if (ex < 0) continue;
      const float gs = gl[s];
      const int mine = lpos[s], first = ebase[ex], last = first + tot[ex];
      int rank = 0;
      for (int j = first; j < last; ++j) {
        const float g2 = lg[j];
        rank += (g2 > gs || (g2 == gs && j < mine)) ? 1 : 0;
      }
      const int64_t t = base + s;
      const bool ok = rank < C;
      pos[t * 2] = rank;
      kept[t * 2] = ok ? 1 : 0;
      if (!ok) gate[t * 2] = gs * 0.0f;
    }
  }
  // tokens that did not compete: mask_k_flat = 0 -> gate_k * 0, kept = 0
  for (int s = tid; s < S; s += CAP_THREADS) {
    int64_t t = base + s;
    if (c1[s] < 0) { kept[t * 2] = 0; gate[t * 2] = gate[t * 2] * 0.0f; }
    if (c2[s] < 0) {
      kept[t * 2 + 1] = 0;
      gate[t * 2 + 1] = gate[t * 2 + 1] * 0.0f;
    }
  }
  if (loss2) {
    cnt[chunk * el + e] = cap_count(c2l, s_begin, s_end, e, vec);
    __syncthreads();
    if (chunk == 0 && e < E) {
      int total = 0;
      for (int k = 0; k < nchunks; ++k) total += cnt[k * el + e];
      tot[2 * el + e] = total;
    }
    __syncthreads();
  }
  // per-expert outputs and the group's share of the balancing loss.  The
  // per-block partial sums of the select step are summed in block order; they
  // come through LDS (`cnt` is free now), nchunks blocks at a time, so that
  // the loads of one batch fly together instead of one after the other.
  float* stage = reinterpret_cast<float*>(cnt);          // [nchunks][el]
  auto sum_blocks = [&](const float* part) {
    float acc = 0.f;
    for (int b0 = 0; b0 < p.nblk; b0 += nchunks) {
      const int bb = b0 + chunk;
      const float v = (bb < p.nblk && e < E)
                          ? part[((int64_t)g * p.nblk + bb) * E + e] : 0.f;
      __syncthreads();
      stage[chunk * el + e] = v;
      __syncthreads();
      if (tid < E)
        for (int k = 0; k < nchunks && b0 + k < p.nblk; ++k)
          acc += stage[k * el + tid];
    }
    return acc;                                          // valid for tid < E
  };
  const float proxy = sum_blocks(part1);
  float proxy2 = 0.f, zsum = 0.f, n_one_sum = 0.f;
  if (loss2 && !sw) proxy2 = sum_blocks(part2);
  if (sw) {
    // columns 0 and 1 of part2: sum of logsumexp^2 and the number of tokens of
    // importance 1; thread e sums column e
    const float colsum = sum_blocks(part2);
    __syncthreads();
    if (tid < 2) stage[tid] = colsum;
    __syncthreads();
    zsum = stage[0];
    n_one_sum = E > 1 ? stage[1] : 0.f;
    __syncthreads();
  }
  if (tid < E) {
    const int t1 = tot[tid], t2 = tot[el + tid];
    const int k1 = min(t1, C);
    fill[(int64_t)g * E + tid] = k1 + min(t2, C - k1);
    const float inv_s = (float)(1.0 / (double)S);
    // density_1: competing first choices (top-2, moe.py:1420-1423) or every
    // token's arg-max (switch, moe.py:1224-1225)
    const int dens = sw ? tot[2 * el + tid] : t1;
    prod[tid] = (proxy * inv_s) * ((float)dens * inv_s);
    if (loss2 && !sw)
      prod[el + tid] = (proxy2 * inv_s) * ((float)tot[2 * el + tid] * inv_s);
  }
  __syncthreads();
  if (tid == 0) {
    float s1 = 0.f, s2 = 0.f;
    for (int k = 0; k < E; ++k) s1 += prod[k];
    if (loss2 && !sw)
      for (int k = 0; k < E; ++k) s2 += prod[el + k];
    gsum[g * GSUM] = s1;
    gsum[g * GSUM + 1] = s2;
    gsum[g * GSUM + 2] = sw ? n_one_sum : 0.f;
    gsum[g * GSUM + 3] = sw ? zsum : 0.f;
  }
}

// The balancing loss from the groups' terms; one thread.  COHERENT: the terms
// were written by other blocks of the same launch (see st_dev).
template <bool COHERENT>
__device__ __forceinline__ void gate_loss_value(const GateParams& p,
                                                const float* gsum_in,
                                                float* loss) {
  struct Terms {
    const float* q;
    __device__ float operator[](int i) const {
      return COHERENT ? ld_dev(q + i) : q[i];
    }
  } gsum = {gsum_in};
  float s1 = 0.f, s2 = 0.f;
  for (int g = 0; g < p.G; ++g) {
    s1 += gsum[g * GSUM];
    s2 += gsum[g * GSUM + 1];
  }
  const float inv_ge = (float)(1.0 / ((double)p.G * (double)p.E));
  const float ee = (float)((double)p.E * (double)p.E);
  float l;
  if (p.router == ROUTER_SWITCH) {
    if (p.has_importance) {
      // mean over [G,E,S] of proxy[g,e] * (imp[g,s] == 1) * density[g,e]
      // (moe.py:1229-1234): each group's term counts once per such token
      float sm = 0.f;
      for (int g = 0; g < p.G; ++g) sm += gsum[g * GSUM] * gsum[g * GSUM + 2];
      l = (sm * (float)(1.0 / ((double)p.G * (double)p.E * (double)p.S))) * ee;
    } else {
      l = (s1 * inv_ge) * ee;
    }
    if (p.num_microbatches > 1)
      l = l * (float)(1.0 / (double)p.num_microbatches);     // moe.py:1235-1238
    if (p.use_z_loss) {                                      // moe.py:1253-1266
      float z = 0.f, n = 0.f;
      for (int g = 0; g < p.G; ++g) {
        z += gsum[g * GSUM + 3];
        n += gsum[g * GSUM + 2];
      }
      const float mb = (float)(p.num_microbatches > 0 ? p.num_microbatches : 1);
      l = l + p.z_loss_coef * (z / (n * mb));
    }
    loss[0] = l;
    return;
  }
  l = (s1 * inv_ge) * ee;                                    // moe.py:1423-1424
  if (p.use_second_place_loss) l = l + ((s2 * inv_ge) * ee) * 0.5f;
  if (p.num_microbatches > 1)
    l = l * (float)(1.0 / (double)p.num_microbatches);       // moe.py:1439-1442
  loss[0] = l;
}

__global__ void gate_loss_kernel(GateParams p, const float* __restrict__ gsum,
                                 float* __restrict__ loss) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  gate_loss_value<false>(p, gsum, loss);
}

static int gate_tokens_per_block(int E) {
  if (E <= 128) return 256;
  if (E <= 256) return 128;
  return 64;
}

}  // namespace mesh_moe

using namespace mesh_moe;

template <int NT>
static int launch_router_mfma(const bf16_t* x, const bf16_t* wp,
                              const float* bias, float* logits, int batch,
                              int tokens, int M, int E, hipStream_t st) {
  const size_t smem = 3 * (128 * 128 + (size_t)NT * 32 * 128);
  auto k = router_mfma_kernel<NT>;
  MOE_ALLOW_LDS(k, smem);
  dim3 grid((unsigned)((tokens + 127) / 128), (unsigned)batch);
  k<<<grid, 256, smem, st>>>(x, wp, bias, logits, tokens, M, E);
  MOE_CHECK_LAUNCH("router_logits (mfma)");
  return 0;
}

extern "C" int mesh_moe_router_logits(const void* x, const void* w,
                                      const void* w_packed, const float* bias,
                                      float* logits, int batch, int64_t tokens,
                                      int M, int E, int dtype, void* stream) {
  MOE_REQUIRE(x && w && logits, MESH_MOE_E_ARG, "router_logits: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "router_logits: bad dtype %d",
              dtype);
  MOE_REQUIRE(batch >= 1 && tokens >= 0 && M >= 1 && E >= 1, MESH_MOE_E_ARG,
              "router_logits: bad sizes batch=%d tokens=%lld M=%d E=%d", batch,
              (long long)tokens, M, E);
  MOE_REQUIRE(E <= 4 * RL_MAX_EPT, MESH_MOE_E_UNSUPPORTED,
              "router_logits: E=%d > %d", E, 4 * RL_MAX_EPT);
  MOE_REQUIRE(batch <= 65535, MESH_MOE_E_UNSUPPORTED,
              "router_logits: batch=%d > 65535", batch);
  if (tokens == 0) return 0;
  if (dtype == MESH_MOE_BF16 && w_packed != nullptr && M % 64 == 0 &&
      E % 4 == 0 && tokens * (int64_t)M < (1LL << 31) &&
      (((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)logits) % 16 == 0)) {
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w_packed;
    hipStream_t s2 = (hipStream_t)stream;
    if (E <= 32)
      return launch_router_mfma<1>(xb, wp, bias, logits, batch, (int)tokens, M, E, s2);
    if (E <= 64)
      return launch_router_mfma<2>(xb, wp, bias, logits, batch, (int)tokens, M, E, s2);
    return launch_router_mfma<4>(xb, wp, bias, logits, batch, (int)tokens, M, E, s2);
  }
  const int ept = (E + 3) / 4;
  dim3 grid((unsigned)((tokens + RL_TOK - 1) / RL_TOK), (unsigned)batch);
  int eptp = 1;
  while (eptp < ept) eptp *= 2;
  size_t smem = sizeof(float) * (RL_TOK * (RL_KC + 1) + (size_t)RL_KC * E + 4 * eptp);
  hipStream_t st = (hipStream_t)stream;
#define MOE_ROUTER_LOGITS(T, P)                                                \
  do {                                                                         \
    auto kern = router_logits_kernel<T, P>;                                    \
    MOE_ALLOW_LDS(kern, smem);                                                 \
    kern<<<grid, 256, smem, st>>>((const T*)x, (const T*)w, bias, logits,      \
                                  tokens, M, E, ept);                          \
  } while (0)
#define MOE_ROUTER_LOGITS_T(T)                                                 \
  switch (eptp) {                                                              \
    case 1: MOE_ROUTER_LOGITS(T, 1); break;                                    \
    case 2: MOE_ROUTER_LOGITS(T, 2); break;                                    \
    case 4: MOE_ROUTER_LOGITS(T, 4); break;                                    \
    case 8: MOE_ROUTER_LOGITS(T, 8); break;                                    \
    case 16: MOE_ROUTER_LOGITS(T, 16); break;                                  \
    default: MOE_ROUTER_LOGITS(T, 32); break;                                  \
  }
  if (dtype == MESH_MOE_F32) {
    MOE_ROUTER_LOGITS_T(float);
  } else {
    MOE_ROUTER_LOGITS_T(bf16_t);
  }
#undef MOE_ROUTER_LOGITS_T
#undef MOE_ROUTER_LOGITS
  MOE_CHECK_LAUNCH("router_logits");
  return 0;
}

// Gating steps 2 and 3 (capacity positions, balancing loss) for every group.
static int launch_capacity_and_loss(const GateParams& p, int32_t* idx,
                                    int32_t* pos, float* gate, uint8_t* kept,
                                    int32_t* fill, float* loss,
                                    const float* part1, const float* part2,
                                    float* gsum, hipStream_t st) {
  int el = 2;
  while (el < p.E) el *= 2;
  size_t smem = sizeof(int32_t) * (2 * CAP_THREADS + 3 * (size_t)el) +
                sizeof(float) * 2 * (size_t)el +
                sizeof(int16_t) * (3 * (size_t)p.S + 1) +
                (p.rank_by_gate ? sizeof(float) * (3 * (size_t)p.S + el) : 0);
  MOE_ALLOW_LDS(gate_capacity_kernel, smem);
  gate_capacity_kernel<<<p.G, CAP_THREADS, smem, st>>>(
      p, idx, pos, gate, kept, fill, part1, part2, gsum, el);
  MOE_CHECK_LAUNCH("gate_capacity");
  gate_loss_kernel<<<1, 64, 0, st>>>(p, gsum, loss);
  MOE_CHECK_LAUNCH("gate_loss");
  return 0;
}

static int check_gating_args(int G, int S, int E, int C, int policy,
                             const float* second_uniform,
                             const void* importance, int importance_dtype,
                             size_t workspace_bytes) {
  MOE_REQUIRE(G >= 1 && S >= 1 && C >= 1, MESH_MOE_E_ARG,
              "top2_gating: bad sizes G=%d S=%d C=%d", G, S, C);
  MOE_REQUIRE(E >= 2 && E <= 512, MESH_MOE_E_UNSUPPORTED,
              "top2_gating: E=%d outside [2, 512]", E);
  MOE_REQUIRE(S <= GATE_MAX_GROUP, MESH_MOE_E_UNSUPPORTED,
              "top2_gating: group size S=%d > %d", S, GATE_MAX_GROUP);
  MOE_REQUIRE(G <= 65535, MESH_MOE_E_UNSUPPORTED, "top2_gating: G=%d > 65535",
              G);
  MOE_REQUIRE(policy >= MESH_MOE_SECOND_ALL && policy <= MESH_MOE_SECOND_RANDOM,
              MESH_MOE_E_ARG, "top2_gating: unknown policy %d", policy);
  MOE_REQUIRE(policy != MESH_MOE_SECOND_RANDOM || second_uniform,
              MESH_MOE_E_ARG,
              "top2_gating: policy RANDOM needs second_uniform samples");
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "top2_gating: bad importance dtype %d", importance_dtype);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_gating_workspace_bytes(G, S, E),
              MESH_MOE_E_ARG, "top2_gating: workspace too small (%zu < %zu)",
              workspace_bytes, mesh_moe_gating_workspace_bytes(G, S, E));
  return 0;
}

static GateParams make_gate_params(int G, int S, int E, int C, int policy,
                                   double threshold, int use_second_place_loss,
                                   int num_microbatches,
                                   int importance_from_slot_gate, int tt) {
  GateParams p;
  p.G = G; p.S = S; p.E = E; p.C = C;
  p.policy = policy;
  p.threshold = (float)threshold;
  p.inv_threshold = (float)(1.0 / (threshold > 1e-9 ? threshold : 1e-9));
  p.use_second_place_loss = use_second_place_loss ? 1 : 0;
  p.num_microbatches = num_microbatches;
  p.importance_from_slot_gate = importance_from_slot_gate ? 1 : 0;
  p.tt = tt;
  p.nblk = (S + tt - 1) / tt;
  p.router = ROUTER_TOP2;
  p.has_importance = 0;
  p.use_z_loss = 0;
  p.z_loss_coef = 0.f;
  p.rank_by_gate = 0;
  return p;
}

static GateParams make_switch_params(int G, int S, int E, int C,
                                     const void* importance, int slots_by_gate,
                                     int use_z_loss, double z_loss_coef,
                                     int num_microbatches, int tt) {
  GateParams p = make_gate_params(G, S, E, C, MESH_MOE_SECOND_NONE, 0.0, 0,
                                  num_microbatches, 0, tt);
  p.router = ROUTER_SWITCH;
  p.has_importance = importance != nullptr;
  p.use_z_loss = use_z_loss ? 1 : 0;
  p.z_loss_coef = (float)z_loss_coef;
  p.rank_by_gate = slots_by_gate ? 1 : 0;
  return p;
}

// LDS the last block of a group needs (gate_group_tail).
static size_t fused_tail_lds_bytes(int nblk, int E) {
  return (((size_t)nblk * E * 4 + 15) & ~(size_t)15) +
         sizeof(int32_t) * 3 * (size_t)E + sizeof(float) * (2 * (size_t)E + 8);
}

template <int NT, typename IT>
static int launch_router_gate(const bf16_t* x, const bf16_t* wp,
                              const float* bias, float* logits, int64_t tokens,
                              int M, const void* importance,
                              const float* second_uniform, const GateParams& p,
                              int32_t* idx, int32_t* pos, float* gate,
                              uint8_t* kept, float* part1, float* part2,
                              int tokens_per_batch, const FusedTail& ft,
                              hipStream_t st) {
  const size_t ring = 3 * (128 * 128 + (size_t)NT * 32 * 128);
  // logits tile, importance flags, choices, per-wavefront counts, column sums
  const size_t tile = sizeof(float) * (128 * (size_t)(p.E + 4) + 128) +
                      3 * 128 * sizeof(int16_t) +
                      6 * (size_t)p.E * sizeof(int32_t) +
                      4 * (size_t)p.E * sizeof(float);
  size_t smem = ring > tile ? ring : tile;
  if (ft.bcnt != nullptr) {
    const size_t tail = fused_tail_lds_bytes(p.nblk, p.E);
    smem = smem > tail ? smem : tail;
  }
  auto k = router_gate_kernel<NT, IT>;
  MOE_ALLOW_LDS(k, smem);
  k<<<(unsigned)(tokens / 128), 256, smem, st>>>(
      x, wp, bias, logits, tokens, M, (const IT*)importance, second_uniform, p,
      idx, pos, gate, kept, part1, part2, tokens_per_batch, ft);
  MOE_CHECK_LAUNCH("router_gate");
  return 0;
}

// Workspace: per-block partial sums of the loss (2 float arrays), the groups'
// terms, and for the single-launch kernel per-block counts (3 int32 arrays)
// and the arrival counters.
extern "C" size_t mesh_moe_gating_workspace_bytes(int G, int S, int E) {
  if (G < 1 || S < 1 || E < 1) return 0;
  const size_t nblk = (size_t)(S + 63) / 64;  // smallest token block of any path
  return sizeof(float) * (2 * (size_t)G * nblk * E + GSUM * (size_t)G) +
         sizeof(int32_t) * 3 * (size_t)G * nblk * E +
         sizeof(unsigned long long) * ((size_t)G + 1) + 3 * 256;
}

// Gating from logits: step 1 (softmax / choices) then steps 2 and 3.
static int run_gating(const GateParams& p, const float* logits,
                      const void* importance, int importance_dtype,
                      const float* second_uniform, int32_t* idx, int32_t* pos,
                      float* gate, uint8_t* kept, int32_t* fill, float* loss,
                      void* workspace, hipStream_t st) {
  const int G = p.G, E = p.E;
  uintptr_t wsp = ((uintptr_t)workspace + 255) & ~(uintptr_t)255;
  float* part1 = (float*)wsp;
  float* part2 = part1 + (size_t)G * p.nblk * E;
  float* gsum = part2 + (size_t)G * p.nblk * E;
  dim3 grid((unsigned)p.nblk, (unsigned)G);
  size_t smem = sizeof(float) * ((size_t)p.tt * (E + 1) + p.tt);
  if (importance && importance_dtype == MESH_MOE_BF16) {
    auto k = gate_select_kernel<bf16_t>;
    MOE_ALLOW_LDS(k, smem);
    k<<<grid, p.tt, smem, st>>>(logits, (const bf16_t*)importance,
                                second_uniform, p, idx, pos, gate, kept, part1,
                                part2);
  } else {
    auto k = gate_select_kernel<float>;
    MOE_ALLOW_LDS(k, smem);
    k<<<grid, p.tt, smem, st>>>(logits, (const float*)importance,
                                second_uniform, p, idx, pos, gate, kept, part1,
                                part2);
  }
  MOE_CHECK_LAUNCH("gate_select");
  return launch_capacity_and_loss(p, idx, pos, gate, kept, fill, loss, part1,
                                  part2, gsum, st);
}

// Number of a single-launch gating call: the arrival counters in the
// workspace are read relative to it (see arrive_is_last).
static unsigned long long next_call_number() {
  static std::atomic<unsigned long long> counter{1};
  unsigned long long n = counter.fetch_add(1, std::memory_order_relaxed);
  return (n & ((1ull << 48) - 1)) | (1ull << 47);
}

// Shape limits of the fused projection + gating kernel.
static int check_fused_router_args(const char* who, const void* x,
                                   const void* w_packed, int batch,
                                   int64_t tokens, int M, int dtype, int G,
                                   int S, int E) {
  MOE_REQUIRE(batch >= 1 && (int64_t)batch * tokens == (int64_t)G * S,
              MESH_MOE_E_ARG, "%s: batch*tokens=%lld != G*S=%lld", who,
              (long long)batch * tokens, (long long)G * S);
  // (the one-launch tail keeps per-block slot prefixes in 16 bits)
  MOE_REQUIRE(S <= GATE_MAX_GROUP, MESH_MOE_E_UNSUPPORTED,
              "%s: group size S=%d > %d", who, S, GATE_MAX_GROUP);
  MOE_REQUIRE(dtype == MESH_MOE_BF16 && M % 64 == 0 && E % 4 == 0 && E <= 128 &&
                  S % 128 == 0 && tokens % S == 0 &&
                  (int64_t)128 * M < (1LL << 31) &&
                  (((uintptr_t)x | (uintptr_t)w_packed) % 16 == 0),
              MESH_MOE_E_UNSUPPORTED,
              "%s: the fused kernel needs bf16, M %% 64 == 0, "
              "E %% 4 == 0, E <= 128, S %% 128 == 0 (M=%d E=%d S=%d dtype=%d); "
              "use router_logits + the logits-in gating call", who, M, E, S,
              dtype);
  return 0;
}

// Fused projection + gating step 1 (p.tt must be 128), then steps 2 and 3.
static int run_router_gating(const GateParams& p, const void* x,
                             const void* w_packed, const float* bias,
                             float* logits, int64_t tokens, int M,
                             const void* importance, int importance_dtype,
                             const float* second_uniform, int32_t* idx,
                             int32_t* pos, float* gate, uint8_t* kept,
                             int32_t* fill, float* loss, void* workspace,
                             hipStream_t st) {
  const int G = p.G, S = p.S, E = p.E;
  uintptr_t wsp = ((uintptr_t)workspace + 255) & ~(uintptr_t)255;
  float* part1 = (float*)wsp;
  float* part2 = part1 + (size_t)G * p.nblk * E;
  float* gsum = part2 + (size_t)G * p.nblk * E;
  const bf16_t* xb = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)w_packed;
  const int64_t total = (int64_t)G * S;
  const bool imp_bf16 = importance && importance_dtype == MESH_MOE_BF16;
  // Slots in token order: positions, fill and loss are finished inside the
  // same launch by the last block of each group.  Slots by gate (switch_max)
  // compare every pair of a group's tokens: the capacity kernel does that.
  FusedTail ft = {};
  const bool one_launch =
      !p.rank_by_gate && fused_tail_lds_bytes(p.nblk, E) <= 60 * 1024;
  if (one_launch) {
    auto up = [](uintptr_t q) { return (q + 255) & ~(uintptr_t)255; };
    ft.bcnt = (int32_t*)up((uintptr_t)(gsum + GSUM * (size_t)G));
    ft.gctr = (unsigned long long*)up(
        (uintptr_t)(ft.bcnt + 3 * (size_t)G * p.nblk * E));
    ft.fctr = ft.gctr + G;
    ft.gsum = gsum;
    ft.fill = fill;
    ft.loss = loss;
    ft.call = next_call_number();
  }
  int rc;
#define MOE_ROUTER_GATE(NT)                                                    \
  (imp_bf16 ? launch_router_gate<NT, bf16_t>(xb, wp, bias, logits, total, M,   \
                                             importance, second_uniform, p,    \
                                             idx, pos, gate, kept, part1,      \
                                             part2, (int)tokens, ft, st)       \
            : launch_router_gate<NT, float>(xb, wp, bias, logits, total, M,    \
                                            importance, second_uniform, p,     \
                                            idx, pos, gate, kept, part1,       \
                                            part2, (int)tokens, ft, st))
  if (E <= 32) rc = MOE_ROUTER_GATE(1);
  else if (E <= 64) rc = MOE_ROUTER_GATE(2);
  else rc = MOE_ROUTER_GATE(4);
#undef MOE_ROUTER_GATE
  if (rc != 0 || one_launch) return rc;
  return launch_capacity_and_loss(p, idx, pos, gate, kept, fill, loss, part1,
                                  part2, gsum, st);
}

// ---------------------------------------------------------------------------
// Scratch memory of mesh_moe_top2_gating_static_scratch: what the other gating
// calls take from the caller as `workspace`.  Every GPU holds its own copy of
// the array at its own address; in host code the array's name is only a
// handle for hipGetSymbolAddress, never a device address.
// ---------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)MESH_MOE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[STATIC_SCRATCH_MAX_DEVICES] = {};

// Device address of `scratch` on the current device, looked up once per
// device; nullptr (error text set) if the runtime refuses.
static void* static_scratch_address() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= STATIC_SCRATCH_MAX_DEVICES) {
    mesh_moe::set_error("static scratch: hipGetDevice gave device %d (%s)", dev,
                        hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      mesh_moe::set_error("static scratch: hipGetSymbolAddress: %s",
                          hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

extern "C" int mesh_moe_top2_gating_static_scratch(
    const float* logits, const void* importance, int importance_dtype,
    int importance_from_slot_gate, const float* second_uniform, int G, int S,
    int E, int C, int policy, double threshold, int use_second_place_loss,
    int num_microbatches, int32_t* idx, int32_t* pos, float* gate,
    uint8_t* kept, int32_t* fill, float* loss, void* stream) {
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1, MESH_MOE_E_ARG,
              "top2_gating_static_scratch: bad sizes G=%d S=%d E=%d", G, S, E);
  const size_t need = mesh_moe_gating_workspace_bytes(G, S, E);
  MOE_REQUIRE(need <= STATIC_SCRATCH_BYTES, MESH_MOE_E_UNSUPPORTED,
              "top2_gating_static_scratch: G=%d S=%d E=%d needs %zu bytes of "
              "scratch, the built-in buffer has %zu; use mesh_moe_top2_gating "
              "with a workspace", G, S, E, need, STATIC_SCRATCH_BYTES);
  void* ptr = static_scratch_address();
  if (ptr == nullptr) return MESH_MOE_E_HIP;
  return mesh_moe_top2_gating(logits, importance, importance_dtype,
                              importance_from_slot_gate, second_uniform, G, S,
                              E, C, policy, threshold, use_second_place_loss,
                              num_microbatches, idx, pos, gate, kept, fill,
                              loss, ptr, STATIC_SCRATCH_BYTES, stream);
}

extern "C" int mesh_moe_top2_gating(
    const float* logits, const void* importance, int importance_dtype,
    int importance_from_slot_gate, const float* second_uniform, int G, int S,
    int E, int C, int policy,
    double threshold, int use_second_place_loss, int num_microbatches,
    int32_t* idx, int32_t* pos, float* gate, uint8_t* kept, int32_t* fill,
    float* loss, void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && idx && pos && gate && kept && fill && loss && workspace,
              MESH_MOE_E_ARG, "top2_gating: null pointer");
  if (int rc = check_gating_args(G, S, E, C, policy, second_uniform, importance,
                                 importance_dtype, workspace_bytes))
    return rc;
  GateParams p = make_gate_params(G, S, E, C, policy, threshold,
                                  use_second_place_loss, num_microbatches,
                                  importance_from_slot_gate,
                                  gate_tokens_per_block(E));
  return run_gating(p, logits, importance, importance_dtype, second_uniform,
                    idx, pos, gate, kept, fill, loss, workspace,
                    (hipStream_t)stream);
}

extern "C" int mesh_moe_router_top2_gating(
    const void* x, const void* w_packed, const float* bias, float* logits,
    int batch, int64_t tokens, int M, int dtype, const void* importance,
    int importance_dtype, int importance_from_slot_gate,
    const float* second_uniform, int G, int S, int E, int C, int policy,
    double threshold, int use_second_place_loss, int num_microbatches,
    int32_t* idx, int32_t* pos, float* gate, uint8_t* kept, int32_t* fill,
    float* loss, void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(x && w_packed && idx && pos && gate && kept && fill && loss &&
                  workspace, MESH_MOE_E_ARG, "router_top2_gating: null pointer");
  if (int rc = check_gating_args(G, S, E, C, policy, second_uniform, importance,
                                 importance_dtype, workspace_bytes))
    return rc;
  if (int rc = check_fused_router_args("router_top2_gating", x, w_packed, batch,
                                       tokens, M, dtype, G, S, E))
    return rc;
  GateParams p = make_gate_params(G, S, E, C, policy, threshold,
                                  use_second_place_loss, num_microbatches,
                                  importance_from_slot_gate, 128);
  return run_router_gating(p, x, w_packed, bias, logits, tokens, M, importance,
                           importance_dtype, second_uniform, idx, pos, gate,
                           kept, fill, loss, workspace, (hipStream_t)stream);
}

extern "C" int mesh_moe_switch_gating(
    const float* logits, const float* choice_logits, const void* importance,
    int importance_dtype, int G, int S, int E, int C, int slots_by_gate,
    int use_z_loss, double z_loss_coef,
    int num_microbatches, int32_t* idx, int32_t* pos, float* gate,
    uint8_t* kept, int32_t* fill, float* loss, void* workspace,
    size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && idx && pos && gate && kept && fill && loss && workspace,
              MESH_MOE_E_ARG, "switch_gating: null pointer");
  if (int rc = check_gating_args(G, S, E, C, MESH_MOE_SECOND_NONE, nullptr,
                                 importance, importance_dtype, workspace_bytes))
    return rc;
  GateParams p = make_switch_params(G, S, E, C, importance, slots_by_gate,
                                    use_z_loss, z_loss_coef, num_microbatches,
                                    gate_tokens_per_block(E));
  return run_gating(p, logits, importance, importance_dtype, choice_logits,
                    idx, pos, gate, kept, fill, loss, workspace,
                    (hipStream_t)stream);
}

extern "C" int mesh_moe_router_switch_gating(
    const void* x, const void* w_packed, const float* bias, float* logits,
    int batch, int64_t tokens, int M, int dtype, const void* importance,
    int importance_dtype, int G, int S, int E, int C, int slots_by_gate,
    int use_z_loss, double z_loss_coef, int num_microbatches, int32_t* idx,
    int32_t* pos,
    float* gate, uint8_t* kept, int32_t* fill, float* loss, void* workspace,
    size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(x && w_packed && idx && pos && gate && kept && fill && loss &&
                  workspace, MESH_MOE_E_ARG,
              "router_switch_gating: null pointer");
  if (int rc = check_gating_args(G, S, E, C, MESH_MOE_SECOND_NONE, nullptr,
                                 importance, importance_dtype, workspace_bytes))
    return rc;
  if (int rc = check_fused_router_args("router_switch_gating", x, w_packed,
                                       batch, tokens, M, dtype, G, S, E))
    return rc;
  GateParams p = make_switch_params(G, S, E, C, importance, slots_by_gate,
                                    use_z_loss, z_loss_coef, num_microbatches,
                                    128);
  return run_router_gating(p, x, w_packed, bias, logits, tokens, M, importance,
                           importance_dtype, nullptr, idx, pos, gate, kept,
                           fill, loss, workspace, (hipStream_t)stream);
}
