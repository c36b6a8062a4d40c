// "No token left behind" gating for gfx950.
//
// Follows _ntlb_gating, mesh_tensorflow/transformer/moe.py:804-940, after the
// router projection: softmax in the operation order of mtf.softmax
// (ops.py:5493-5541) and in the dtype the reference runs it in -- this router
// alone keeps the projection's result and the softmax in the activation dtype
// and casts the probabilities to float32 afterwards (moe.py:825-836), so with
// bfloat16 activations every op of the chain rounds to bfloat16 --, the top_k
// experts of every token (mtf.top_k,
// ops.py:4964-5015: repeated first-arg-max), then top_k passes in which the
// still unrouted tokens are offered, in token order, to their next expert
// (moe.py:903-934).  The dense [G,S,k,E] masks and the cumsum over the group
// are replaced by per-token candidate lists and integer counting; the result
// is the [G,S,2] routing record of the other routers with the second choice
// never kept.
#include "common.h"

namespace mesh_moe {

constexpr int NTLB_MAX_K = 8;
constexpr int NTLB_THREADS = 1024;
constexpr int NTLB_GSUM = 2;  // floats per group: loss term, #(importance == 1)

struct NtlbParams {
  int G, S, E, C, K;
  int num_microbatches;
  int has_importance;
  int tt;    // tokens per block of the select kernel
  int nblk;  // its blocks per group
};

// ---------------------------------------------------------------------------
// Step 1: one thread per token.  Softmax, the K best experts (ties: lowest
// index), the candidates' probabilities; per block column sums of the
// probabilities (density_1_proxy, moe.py:848) and the number of tokens with
// importance 1.
// ---------------------------------------------------------------------------
// The probabilities of one row in place, ST = dtype of the reference's softmax
// ops.  ST = bf16_t: the logits are first rounded (the projection's bfloat16
// result), then every op rounds once (negative and max are exact; the sum
// accumulates in float32 in index order and rounds once, as TensorFlow's
// bfloat16 sum reducer does).  ST = float: round_to is the identity.
template <typename ST>
__device__ __forceinline__ void ntlb_softmax_row(float* row, int E) {
  for (int e = 0; e < E; ++e) row[e] = round_to<ST>(row[e]);
  float m = row[0];
  for (int e = 1; e < E; ++e) m = fmaxf(m, row[e]);       // reduce_max
  const float negm = -m;
  float s = 0.f;                                          // exp, reduce_sum
  for (int e = 0; e < E; ++e)
    s += round_to<ST>(expf(round_to<ST>(row[e] + negm)));
  s = round_to<ST>(s);
  const float neglse = -round_to<ST>(round_to<ST>(logf(s)) + m);  // log + max
  for (int e = 0; e < E; ++e)
    row[e] = round_to<ST>(expf(round_to<ST>(row[e] + neglse)));
}

template <typename IT, typename ST>
__global__ __launch_bounds__(256) void ntlb_select_kernel(
    NtlbParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, int16_t* __restrict__ cand_idx,
    float* __restrict__ cand_gate, uint8_t* __restrict__ competes,
    float* __restrict__ part, float* __restrict__ part_one) {
  extern __shared__ float smem[];
  const int E = p.E, S = p.S, K = p.K;
  const int ld = E + 1;
  float* tile = smem;                          // [tt][E+1]
  float* isone = smem + (size_t)p.tt * ld;     // [tt]
  const int g = blockIdx.y, blk = blockIdx.x;
  const int t0 = blk * p.tt;
  const int ntok = min(p.tt, S - t0);
  const int tid = threadIdx.x;
  const float* src = logits + ((int64_t)g * S + t0) * E;
  for (int i = tid; i < ntok * E; i += blockDim.x) {
    int r = i / E, c = i - r * E;
    tile[r * ld + c] = src[i];
  }
  __syncthreads();
  if (tid < ntok) {
    float* row = tile + tid * ld;
    const int64_t t = (int64_t)g * S + t0 + tid;
    ntlb_softmax_row<ST>(row, E);
    bool one = true;
    if (importance != nullptr) one = (load_f32<IT>(importance + t) == 1.0f);
    float vals[NTLB_MAX_K];
    int ids[NTLB_MAX_K];
#pragma unroll
    for (int i = 0; i < NTLB_MAX_K; ++i) {
      if (i < K) {
        float best = -1.f;
        int bi = 0;
        for (int e = 0; e < E; ++e) {
          const float v = row[e];
          if (v > best) { best = v; bi = e; }               // first arg-max
        }
        vals[i] = best;
        ids[i] = bi;
        row[bi] = -2.f;                                     // taken
      }
    }
#pragma unroll
    for (int i = 0; i < NTLB_MAX_K; ++i) {
      if (i < K) {
        row[ids[i]] = vals[i];
        cand_idx[t * K + i] = (int16_t)ids[i];
        cand_gate[t * K + i] = one ? vals[i] : vals[i] * 0.0f;  // moe.py:851
      }
    }
    competes[t] = one ? 1 : 0;
    isone[tid] = one ? 1.0f : 0.0f;
  }
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) {
    float s = 0.f;
    for (int r = 0; r < ntok; ++r) s += tile[r * ld + e];
    part[((int64_t)g * p.nblk + blk) * E + e] = s;
  }
  if (tid == 0) {
    float n = 0.f;
    for (int r = 0; r < ntok; ++r) n += isone[r];
    part_one[(int64_t)g * p.nblk + blk] = n;
  }
}

// ---------------------------------------------------------------------------
// Step 2: one block per group.  Thread (e = tid % el, chunk = tid / el), as in
// the capacity kernel of the other routers.  Pass i: every thread counts the
// offers to expert e in its chunk of tokens (unrouted tokens with importance 1
// whose i-th candidate is e), an exclusive prefix over the chunks gives the
// chunk's starting count on top of what the expert holds, and a second walk
// takes the offers whose running count stays within the capacity
// (moe.py:908-916: the count includes the offers that are turned down).  Each
// token is visited by exactly one thread per pass.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(NTLB_THREADS) void ntlb_assign_kernel(
    NtlbParams p, const int16_t* __restrict__ cand_idx,
    const float* __restrict__ cand_gate, const uint8_t* __restrict__ competes,
    const float* __restrict__ part, const float* __restrict__ part_one,
    int32_t* __restrict__ idx, int32_t* __restrict__ pos,
    float* __restrict__ gate, uint8_t* __restrict__ kept,
    int32_t* __restrict__ fill, float* __restrict__ gsum, int el) {
  extern __shared__ __attribute__((aligned(16))) int32_t smem_i[];
  const int S = p.S, E = p.E, C = p.C, K = p.K;
  int32_t* cnt = smem_i;                          // [nchunks][el]
  int32_t* held = cnt + NTLB_THREADS;             // [el]
  int32_t* named = held + el;                     // [K][el] density counts
  float* prod = reinterpret_cast<float*>(named + (size_t)K * el);  // [el]
  int16_t* cand = reinterpret_cast<int16_t*>(prod + el);  // [K][S]
  uint8_t* open_ = reinterpret_cast<uint8_t*>(cand + (size_t)K * S);  // [S]
  // what the passes decide per token, written out in one parallel sweep at
  // the end: the pass that placed it (0xff: none) and its slot
  uint8_t* wpass = open_ + S;                                          // [S]
  int16_t* wpos = reinterpret_cast<int16_t*>(wpass + S + (S & 1));     // [S]
  const int g = blockIdx.x, tid = threadIdx.x;
  const int64_t base = (int64_t)g * S;
  for (int i = tid; i < S * K; i += NTLB_THREADS) {
    const int s = i / K, k = i - s * K;
    cand[k * S + s] = cand_idx[base * K + i];
  }
  for (int s = tid; s < S; s += NTLB_THREADS) {
    open_[s] = competes[base + s];
    wpass[s] = 0xff;
  }
  if (tid < el) held[tid] = 0;
  __syncthreads();
  const int e = tid % el;
  const int chunk = tid / el;
  const int nchunks = NTLB_THREADS / el;
  const int clen = (S + nchunks - 1) / nchunks;
  const int s_begin = min(S, chunk * clen);
  const int s_end = min(S, s_begin + clen);
  // 16-byte reads: every array starts 16-byte aligned and a chunk holds whole
  // groups of eight tokens
  const bool vec = (el % 4 == 0) && (S % 8 == 0) && (clen % 8 == 0);
  for (int i = 0; i < K; ++i) {
    const int16_t* ch = cand + (size_t)i * S;
    // density_1 of this pass counts every token (moe.py:847 precedes the
    // importance mask), the offers only the open ones
    int all = 0, c = 0;
    if (vec) {
      // eight tokens per step: one 16-byte read of the candidates, one 8-byte
      // read of the open flags
      for (int s = s_begin; s < s_end; s += 8) {
        const uint4 c8 = *reinterpret_cast<const uint4*>(ch + s);
        const uint2 o8 = *reinterpret_cast<const uint2*>(open_ + s);
        const uint32_t cw[4] = {c8.x, c8.y, c8.z, c8.w};
        const uint32_t ow[2] = {o8.x, o8.y};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int id = (int)(int16_t)((cw[j >> 1] >> (16 * (j & 1))) & 0xffffu);
          const bool hit = id == e;
          const bool op = ((ow[j >> 2] >> (8 * (j & 3))) & 0xffu) != 0;
          all += hit;
          c += hit && op;
        }
      }
    } else {
      for (int s = s_begin; s < s_end; ++s) {
        const bool hit = ch[s] == e;
        all += hit;
        c += hit && open_[s];
      }
    }
    cnt[chunk * el + e] = c;
    __syncthreads();
    int before = 0, total = 0;
    for (int k = 0; k < nchunks; ++k) {
      const int v = cnt[k * el + e];
      total += v;
      if (k < chunk) before += v;
    }
    const int have = held[e];
    int running = have + before;
    __syncthreads();            // everybody has read cnt and held
    cnt[chunk * el + e] = all;
    // (a token's flags are written by the one thread whose expert is its
    // candidate in this pass, so reading eight of them ahead is safe)
    auto offer = [&](int s) {
      ++running;
      if (running <= C) {
        wpass[s] = (uint8_t)i;
        wpos[s] = (int16_t)(running - 1);
        open_[s] = 0;
      }
    };
    if (vec) {
      for (int s = s_begin; s < s_end; s += 8) {
        const uint4 c8 = *reinterpret_cast<const uint4*>(ch + s);
        const uint2 o8 = *reinterpret_cast<const uint2*>(open_ + s);
        const uint32_t cw[4] = {c8.x, c8.y, c8.z, c8.w};
        const uint32_t ow[2] = {o8.x, o8.y};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int id = (int)(int16_t)((cw[j >> 1] >> (16 * (j & 1))) & 0xffffu);
          const bool op = ((ow[j >> 2] >> (8 * (j & 3))) & 0xffu) != 0;
          if (id == e && op) offer(s + j);
        }
      }
    } else {
      for (int s = s_begin; s < s_end; ++s)
        if (ch[s] == e && open_[s]) offer(s);
    }
    __syncthreads();
    if (chunk == 0) {
      int n = 0;
      for (int k = 0; k < nchunks; ++k) n += cnt[k * el + e];
      named[i * el + e] = n;
      held[e] = min(C, have + total);
    }
    __syncthreads();
  }
  // the records: a placed token names its expert, slot and gate; the others
  // keep their first candidate as a stand-in, not routed
  for (int s = tid; s < S; s += NTLB_THREADS) {
    const int64_t t = base + s;
    const int ps = wpass[s];
    const bool placed = ps != 0xff;
    idx[t * 2] = placed ? (int32_t)cand[(size_t)ps * S + s] : (int32_t)cand[s];
    idx[t * 2 + 1] = 0;
    pos[t * 2] = placed ? (int32_t)wpos[s] : 0;
    pos[t * 2 + 1] = 0;
    gate[t * 2] = placed ? cand_gate[t * K + ps] : 0.0f;
    gate[t * 2 + 1] = 0.0f;
    kept[t * 2] = placed ? 1 : 0;
    kept[t * 2 + 1] = 0;
  }
  if (tid < E) fill[(int64_t)g * E + tid] = held[tid];
  // the group's share of the loss: sum over passes and experts of
  // proxy[e] * density[i][e] (moe.py:848, :854)
  if (tid < E) {
    float proxy = 0.f;
    for (int b = 0; b < p.nblk; ++b)
      proxy += part[((int64_t)g * p.nblk + b) * E + tid];
    prod[tid] = proxy * (float)(1.0 / (double)S);
  }
  __syncthreads();
  if (tid == 0) {
    const float inv_s = (float)(1.0 / (double)S);
    float sum = 0.f;
    for (int i = 0; i < K; ++i)
      for (int k = 0; k < E; ++k)
        sum += prod[k] * ((float)named[i * el + k] * inv_s);
    float n_one = 0.f;
    for (int b = 0; b < p.nblk; ++b) n_one += part_one[(int64_t)g * p.nblk + b];
    gsum[g * NTLB_GSUM] = sum;
    gsum[g * NTLB_GSUM + 1] = n_one;
  }
}

__global__ void ntlb_loss_kernel(NtlbParams p, const float* __restrict__ gsum,
                                 float* __restrict__ loss) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const double terms = (double)p.G * (double)p.K * (double)p.E;
  const float ee = (float)((double)p.E * (double)p.E);
  float s = 0.f, l;
  if (p.has_importance) {
    // the proxy carries (importance == 1) [G,S]: every group's sum counts once
    // per such token and the mean runs over the group dim too (moe.py:849-856)
    for (int g = 0; g < p.G; ++g)
      s += gsum[g * NTLB_GSUM] * gsum[g * NTLB_GSUM + 1];
    l = (s * (float)(1.0 / (terms * (double)p.S))) * ee;
  } else {
    for (int g = 0; g < p.G; ++g) s += gsum[g * NTLB_GSUM];
    l = (s * (float)(1.0 / terms)) * ee;
  }
  if (p.num_microbatches > 1)
    l = l * (float)(1.0 / (double)p.num_microbatches);       // moe.py:857-860
  loss[0] = l;
}

static int ntlb_tokens_per_block(int E) {
  if (E <= 128) return 256;
  if (E <= 256) return 128;
  return 64;
}

}  // namespace mesh_moe

using namespace mesh_moe;

static inline uintptr_t ntlb_up(uintptr_t v) {
  return (v + 255) & ~(uintptr_t)255;
}

extern "C" size_t mesh_moe_ntlb_workspace_bytes(int G, int S, int E,
                                                int top_k) {
  if (G < 1 || S < 1 || E < 1 || top_k < 1) return 0;
  const size_t tok = (size_t)G * S;
  const size_t nblk = ((size_t)S + ntlb_tokens_per_block(E) - 1) /
                      ntlb_tokens_per_block(E);
  return sizeof(int16_t) * tok * top_k + sizeof(float) * tok * top_k + tok +
         sizeof(float) * (size_t)G * nblk * (E + 1) +
         sizeof(float) * (size_t)G * NTLB_GSUM + 6 * 256;
}

extern "C" int mesh_moe_ntlb_gating(
    const float* logits, int softmax_dtype, const void* importance,
    int importance_dtype, int G,
    int S, int E, int C, int top_k, int num_microbatches, int32_t* idx,
    int32_t* pos, float* gate, uint8_t* kept, int32_t* fill, float* loss,
    void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && idx && pos && gate && kept && fill && loss && workspace,
              MESH_MOE_E_ARG, "ntlb_gating: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && C >= 1, MESH_MOE_E_ARG,
              "ntlb_gating: bad sizes G=%d S=%d C=%d", G, S, C);
  MOE_REQUIRE(E >= 2 && E <= 512, MESH_MOE_E_UNSUPPORTED,
              "ntlb_gating: E=%d outside [2, 512]", E);
  MOE_REQUIRE(top_k >= 1 && top_k <= E, MESH_MOE_E_ARG,
              "ntlb_gating: top_k=%d with %d experts", top_k, E);
  MOE_REQUIRE(top_k <= NTLB_MAX_K, MESH_MOE_E_UNSUPPORTED,
              "ntlb_gating: top_k=%d > %d", top_k, NTLB_MAX_K);
  MOE_REQUIRE(S <= 16384 && G <= 65535, MESH_MOE_E_UNSUPPORTED,
              "ntlb_gating: S=%d > 16384 or G=%d > 65535", S, G);
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "ntlb_gating: bad importance dtype %d", importance_dtype);
  MOE_REQUIRE(valid_dtype(softmax_dtype), MESH_MOE_E_ARG,
              "ntlb_gating: bad softmax dtype %d", softmax_dtype);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_ntlb_workspace_bytes(G, S, E, top_k),
              MESH_MOE_E_ARG, "ntlb_gating: workspace too small");
  int el = 2;
  while (el < E) el *= 2;
  const size_t smem2 = sizeof(int32_t) * (NTLB_THREADS + (size_t)el +
                                          (size_t)top_k * el) +
                       sizeof(float) * (size_t)el +
                       sizeof(int16_t) * (size_t)top_k * S + (size_t)S +
                       (size_t)S + 2 + sizeof(int16_t) * (size_t)S;
  MOE_REQUIRE(smem2 <= 160 * 1024, MESH_MOE_E_UNSUPPORTED,
              "ntlb_gating: top_k * S = %d * %d candidates do not fit in LDS",
              top_k, S);
  NtlbParams p;
  p.G = G; p.S = S; p.E = E; p.C = C; p.K = top_k;
  p.num_microbatches = num_microbatches;
  p.has_importance = importance ? 1 : 0;
  p.tt = ntlb_tokens_per_block(E);
  p.nblk = (S + p.tt - 1) / p.tt;
  const size_t tok = (size_t)G * S;
  int16_t* cand_idx = (int16_t*)ntlb_up((uintptr_t)workspace);
  float* cand_gate = (float*)ntlb_up((uintptr_t)(cand_idx + tok * top_k));
  uint8_t* competes = (uint8_t*)ntlb_up((uintptr_t)(cand_gate + tok * top_k));
  float* part = (float*)ntlb_up((uintptr_t)(competes + tok));
  float* part_one = (float*)ntlb_up((uintptr_t)(part + (size_t)G * p.nblk * E));
  float* gsum = (float*)ntlb_up((uintptr_t)(part_one + (size_t)G * p.nblk));
  hipStream_t st = (hipStream_t)stream;
  const size_t smem1 = sizeof(float) * ((size_t)p.tt * (E + 1) + p.tt);
  dim3 grid((unsigned)p.nblk, (unsigned)G);
#define MOE_NTLB_SELECT(IT, ST)                                                \
  do {                                                                         \
    auto k = ntlb_select_kernel<IT, ST>;                                       \
    MOE_ALLOW_LDS(k, smem1);                                                   \
    k<<<grid, 256, smem1, st>>>(p, logits, (const IT*)importance, cand_idx,    \
                                cand_gate, competes, part, part_one);          \
  } while (0)
  const bool imp_bf16 = importance && importance_dtype == MESH_MOE_BF16;
  if (softmax_dtype == MESH_MOE_BF16) {
    if (imp_bf16) MOE_NTLB_SELECT(bf16_t, bf16_t);
    else MOE_NTLB_SELECT(float, bf16_t);
  } else {
    if (imp_bf16) MOE_NTLB_SELECT(bf16_t, float);
    else MOE_NTLB_SELECT(float, float);
  }
#undef MOE_NTLB_SELECT
  MOE_CHECK_LAUNCH("ntlb_gating (select)");
  MOE_ALLOW_LDS(ntlb_assign_kernel, smem2);
  ntlb_assign_kernel<<<G, NTLB_THREADS, smem2, st>>>(
      p, cand_idx, cand_gate, competes, part, part_one, idx, pos, gate, kept,
      fill, gsum, el);
  MOE_CHECK_LAUNCH("ntlb_gating (assign)");
  ntlb_loss_kernel<<<1, 64, 0, st>>>(p, gsum, loss);
  MOE_CHECK_LAUNCH("ntlb_gating (loss)");
  return 0;
}
