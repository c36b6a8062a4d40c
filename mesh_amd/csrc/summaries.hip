// Training-time scalar summaries of the switch, switch-max, ntlb and
// expert-selection routers for gfx950.
//
// The reference emits them with mtf.scalar_summary while training
// (mesh_tensorflow/transformer/moe.py): the mean entropy of the router's
// distribution (:865-868, :1010-1013, :1149-1152, :1242-1245), the mean
// first-choice probability "expert_gate" (:981, :1213), the share of every
// expert among the routed choices "experts/.." (:870-879, :1015-1024,
// :1247-1256), "fraction_routed" (:1041-1046, :1285-1289), the router z-loss
// (:1259-1269) and, for expert selection, how many experts took the token at
// every position of the group "group_token/.." (:1154-1164).  They are
// recomputed here from the float32 logits and the routing record with the
// forward kernels' softmax arithmetic: one thread per token (per-token
// routers) or one block per (group, expert) column (expert selection), per
// block partial sums, and a second kernel that adds the partial sums in a
// fixed order, so the values have the same bits on every run.
#include "common.h"

namespace mesh_moe {

constexpr int SUM_MAX_K = 8;
constexpr int SUM_THREADS = 256;
// floats of a block's partial record before its E per-expert counts
constexpr int SUM_HEAD = 6;
enum { SUM_ENTROPY = 0, SUM_GATE = 1, SUM_KEPT = 2, SUM_IMPORTANCE = 3,
       SUM_LSE2 = 4, SUM_ONES = 5 };

struct SummaryParams {
  int G, S, E, K;
  int router;  // 1 = switch / switch_max, 2 = ntlb
  int tt;      // tokens per block
  int nblk;    // blocks per group
};

template <typename ST>
__device__ __forceinline__ float sum_round(float v) { return round_to<ST>(v); }

// one thread per token; block partial sums to part [G * nblk][SUM_HEAD + E]
template <typename IT, typename ST>
__global__ __launch_bounds__(SUM_THREADS) void router_summary_kernel(
    SummaryParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, const uint8_t* __restrict__ kept,
    float* __restrict__ part) {
  extern __shared__ float sum_smem[];
  const int E = p.E, S = p.S, K = p.K;
  const int ld = E + 1;
  float* tile = sum_smem;                         // [tt][E + 1]
  float* vals = tile + (size_t)p.tt * ld;          // [SUM_HEAD][tt]
  int* hist = reinterpret_cast<int*>(vals + (size_t)SUM_HEAD * p.tt);  // [E]
  const int g = blockIdx.y, blk = blockIdx.x, tid = threadIdx.x;
  const int t0 = blk * p.tt;
  const int ntok = min(p.tt, S - t0);
  const float* src = logits + ((int64_t)g * S + t0) * E;
  for (int i = tid; i < ntok * E; i += blockDim.x) {
    const int r = i / E, c = i - r * E;
    tile[r * ld + c] = src[i];
  }
  for (int e = tid; e < E; e += blockDim.x) hist[e] = 0;
  __syncthreads();
  if (tid < ntok) {
    float* row = tile + tid * ld;
    const int64_t t = (int64_t)g * S + t0 + tid;
    // mtf.softmax (ops.py:5493-5541) in the dtype the router runs it in
    for (int e = 0; e < E; ++e) row[e] = sum_round<ST>(row[e]);
    float m = row[0];
    for (int e = 1; e < E; ++e) m = fmaxf(m, row[e]);
    const float negm = -m;
    float s = 0.f;
    for (int e = 0; e < E; ++e)
      s += sum_round<ST>(expf(sum_round<ST>(row[e] + negm)));
    s = sum_round<ST>(s);
    const float lse = sum_round<ST>(sum_round<ST>(logf(s)) + m);
    const float neglse = -lse;
    float ent = 0.f;
    for (int e = 0; e < E; ++e) {
      const float pe = sum_round<ST>(expf(sum_round<ST>(row[e] + neglse)));
      row[e] = pe;
      ent += -pe * logf(pe + 1e-9f);            // float32 after to_float
    }
    float imp = 1.0f;
    if (importance != nullptr) imp = load_f32<IT>(importance + t);
    const bool one = imp == 1.0f;
    float first = 0.f;
#pragma unroll
    for (int i = 0; i < SUM_MAX_K; ++i) {
      if (i < K) {
        float best = -1.f;
        int bi = 0;
        for (int e = 0; e < E; ++e) {
          const float v = row[e];
          if (v > best) { best = v; bi = e; }     // first arg-max
        }
        if (i == 0) first = best;
        row[bi] = -2.f;
        // expert_mask after "*= (importance == 1)" (moe.py:850, :995, :1228)
        if (one) atomicAdd(&hist[bi], 1);
      }
    }
    vals[SUM_ENTROPY * p.tt + tid] = ent;
    vals[SUM_GATE * p.tt + tid] = first;
    vals[SUM_KEPT * p.tt + tid] = kept != nullptr && kept[t * 2] ? 1.f : 0.f;
    vals[SUM_IMPORTANCE * p.tt + tid] = imp;
    vals[SUM_LSE2 * p.tt + tid] = one ? lse * lse : 0.f;
    vals[SUM_ONES * p.tt + tid] = one ? 1.f : 0.f;
  }
  __syncthreads();
  float* out = part + ((int64_t)g * p.nblk + blk) * (SUM_HEAD + E);
  if (tid < SUM_HEAD) {
    float a = 0.f;
    for (int r = 0; r < ntok; ++r) a += vals[tid * p.tt + r];
    out[tid] = a;
  }
  for (int e = tid; e < E; e += blockDim.x) out[SUM_HEAD + e] = (float)hist[e];
}

// Sum of column c of part [nparts][rec] by one wavefront: lane l adds rows l,
// l + 64, .. in order, then the lanes' sums meet in a fixed butterfly (the same
// bits on every run).
__device__ __forceinline__ float sum_column(const float* __restrict__ part,
                                            int nparts, int rec, int c) {
  const int lane = threadIdx.x & 63;
  float a = 0.f;
  for (int i = lane; i < nparts; i += 64) a += part[(int64_t)i * rec + c];
#pragma unroll
  for (int w = 32; w > 0; w >>= 1) a += __shfl_xor(a, w, 64);
  return a;
}

// out [4 + E]: mean entropy, mean first-choice probability, fraction routed,
// z-loss, then every expert's share of the routed choices.  One block of 16
// wavefronts, a wavefront per column of the partial records.
constexpr int SUM_FINISH_THREADS = 1024;
__global__ __launch_bounds__(SUM_FINISH_THREADS) void router_summary_finish_kernel(
    SummaryParams p, const float* __restrict__ part, int num_microbatches,
    float* __restrict__ out) {
  extern __shared__ float fin[];                  // [SUM_HEAD + E]
  const int nparts = p.G * p.nblk, E = p.E, tid = threadIdx.x;
  const int rec = SUM_HEAD + E;
  const int wave = tid >> 6, lane = tid & 63;
  for (int c = wave; c < rec; c += SUM_FINISH_THREADS / 64) {
    const float a = sum_column(part, nparts, rec, c);
    if (lane == 0) fin[c] = a;
  }
  __syncthreads();
  __shared__ float total;
  if (tid == 0) {
    // the counts are integers: their float sums are exact below 2^24 routed
    // choices, beyond that they round as the reference's reduce_sum does
    float a = 0.f;
    for (int e = 0; e < E; ++e) a += fin[SUM_HEAD + e];
    total = a;
    const float tokens = (float)p.G * (float)p.S;
    out[0] = fin[SUM_ENTROPY] / tokens;
    out[1] = fin[SUM_GATE] / tokens;
    out[2] = fin[SUM_KEPT] / fin[SUM_IMPORTANCE];
    out[3] = fin[SUM_LSE2] /
             (fin[SUM_ONES] * (float)(num_microbatches > 0 ? num_microbatches : 1));
  }
  __syncthreads();
  for (int e = tid; e < E; e += SUM_FINISH_THREADS)
    out[4 + e] = fin[SUM_HEAD + e] / total;
}

// Expert selection: the softmax runs over the group's tokens per expert
// (moe.py:1092-1097, logits of importance-0 tokens lowered by 1e9 first).  One
// block per (expert, group) column: entropy of the column to ent [G * E].
template <typename IT>
__global__ __launch_bounds__(SUM_THREADS) void choice_entropy_kernel(
    int G, int S, int E, const float* __restrict__ logits,
    const IT* __restrict__ importance, float* __restrict__ ent) {
  __shared__ float red[SUM_THREADS];
  const int e = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
  auto value = [&](int s) {
    float x = logits[((int64_t)g * S + s) * E + e];
    if (importance != nullptr &&
        load_f32<IT>(importance + (int64_t)g * S + s) == 0.0f)
      x += 1.0f * -1e9f;
    return x;
  };
  auto block_reduce = [&](float v, bool is_max) {
    red[tid] = v;
    __syncthreads();
    for (int w = SUM_THREADS / 2; w > 0; w >>= 1) {
      if (tid < w)
        red[tid] = is_max ? fmaxf(red[tid], red[tid + w]) : red[tid] + red[tid + w];
      __syncthreads();
    }
    const float r = red[0];
    __syncthreads();
    return r;
  };
  float m = -INFINITY;
  for (int s = tid; s < S; s += SUM_THREADS) m = fmaxf(m, value(s));
  m = block_reduce(m, true);
  float a = 0.f;
  for (int s = tid; s < S; s += SUM_THREADS) a += expf(value(s) - m);
  a = block_reduce(a, false);
  const float neglse = -(logf(a) + m);
  float h = 0.f;
  for (int s = tid; s < S; s += SUM_THREADS) {
    const float pe = expf(value(s) + neglse);
    h += -pe * logf(pe + 1e-9f);
  }
  h = block_reduce(h, false);
  if (tid == 0) ent[(int64_t)g * E + e] = h;
}

// out[0] = mean column entropy; out[4 + s] = (number of (group, expert) pairs
// whose expert took the token at position s) * E * C  (moe.py:1155-1158).
// One wavefront per group position (and wavefront 0 of block 0 for the mean):
// the lanes walk the position's [G][E] entries of tok_slot, integer counts.
__global__ __launch_bounds__(SUM_THREADS) void choice_summary_finish_kernel(
    int G, int S, int E, int C, const float* __restrict__ ent,
    const int16_t* __restrict__ tok_slot, float* __restrict__ out) {
  const int tid = threadIdx.x, lane = tid & 63;
  if (blockIdx.x == 0 && tid < 64) {
    const float a = sum_column(ent, G * E, 1, 0);
    if (lane == 0) {
      out[0] = a / ((float)G * (float)E);
      out[1] = 0.f;
      out[2] = 0.f;
      out[3] = 0.f;
    }
  }
  const int s = blockIdx.x * (SUM_THREADS / 64) + (tid >> 6);
  if (s >= S) return;
  int n = 0;
  for (int i = lane; i < G * E; i += 64) {
    const int g = i / E, e = i - g * E;
    n += tok_slot[((int64_t)g * S + s) * E + e] >= 0 ? 1 : 0;
  }
#pragma unroll
  for (int w = 32; w > 0; w >>= 1) n += __shfl_xor(n, w, 64);
  if (lane == 0) out[4 + s] = (float)n * ((float)E * (float)C);
}

static int summary_tokens_per_block(int E) {
  // logits tile [tt][E + 1] + SUM_HEAD values per token + the histogram
  int tt = SUM_THREADS;
  while (tt > 32 &&
         sizeof(float) * ((size_t)tt * (E + 1 + SUM_HEAD) + E) > 60 * 1024)
    tt >>= 1;
  return tt;
}

}  // namespace mesh_moe

using namespace mesh_moe;

extern "C" size_t mesh_moe_router_summaries_workspace_bytes(int G, int S, int E) {
  if (G < 1 || S < 1 || E < 1) return 0;
  const int tt = summary_tokens_per_block(E);
  const size_t nblk = ((size_t)S + tt - 1) / tt;
  const size_t per_token = sizeof(float) * (size_t)G * nblk * (SUM_HEAD + E);
  const size_t per_column = sizeof(float) * (size_t)G * E;
  return (per_token > per_column ? per_token : per_column) + 256;
}

extern "C" int mesh_moe_router_summaries(
    const float* logits, int softmax_dtype, const void* importance,
    int importance_dtype, const uint8_t* kept, const int16_t* tok_slot, int G,
    int S, int E, int C, int router, int top_k, int num_microbatches,
    float* out, void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && out && workspace, MESH_MOE_E_ARG,
              "router_summaries: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 2 && E <= 512 && G <= 65535 && C >= 1,
              MESH_MOE_E_ARG, "router_summaries: bad sizes G=%d S=%d E=%d C=%d",
              G, S, E, C);
  MOE_REQUIRE(router >= 1 && router <= 3, MESH_MOE_E_ARG,
              "router_summaries: router %d (1 = switch / switch_max, 2 = ntlb, "
              "3 = expert selection; top-2 gating has no summaries)", router);
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "router_summaries: bad importance dtype %d", importance_dtype);
  MOE_REQUIRE(valid_dtype(softmax_dtype), MESH_MOE_E_ARG,
              "router_summaries: bad softmax dtype %d", softmax_dtype);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_router_summaries_workspace_bytes(G, S, E),
              MESH_MOE_E_ARG, "router_summaries: workspace of %zu bytes, need %zu",
              workspace_bytes, mesh_moe_router_summaries_workspace_bytes(G, S, E));
  hipStream_t st = (hipStream_t)stream;
  float* ws = reinterpret_cast<float*>(
      ((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  if (router == 3) {
    MOE_REQUIRE(tok_slot != nullptr, MESH_MOE_E_ARG,
                "router_summaries: expert selection needs tok_slot");
    MOE_REQUIRE(softmax_dtype == MESH_MOE_F32, MESH_MOE_E_ARG,
                "router_summaries: expert selection runs in float32");
    dim3 grid((unsigned)E, (unsigned)G);
    if (importance == nullptr || importance_dtype == MESH_MOE_F32)
      choice_entropy_kernel<float><<<grid, SUM_THREADS, 0, st>>>(
          G, S, E, logits, (const float*)importance, ws);
    else
      choice_entropy_kernel<bf16_t><<<grid, SUM_THREADS, 0, st>>>(
          G, S, E, logits, (const bf16_t*)importance, ws);
    MOE_CHECK_LAUNCH("router_summaries (column entropy)");
    const int per_block = SUM_THREADS / 64;
    choice_summary_finish_kernel<<<(unsigned)((S + per_block - 1) / per_block),
                                   SUM_THREADS, 0, st>>>(G, S, E, C, ws, tok_slot,
                                                         out);
    MOE_CHECK_LAUNCH("router_summaries (finish)");
    return 0;
  }
  MOE_REQUIRE(router != 1 || kept != nullptr, MESH_MOE_E_ARG,
              "router_summaries: the switch routers need kept");
  const int k = router == 2 ? top_k : 1;
  MOE_REQUIRE(k >= 1 && k <= E && k <= SUM_MAX_K, MESH_MOE_E_ARG,
              "router_summaries: top_k=%d with %d experts (at most %d)", k, E,
              SUM_MAX_K);
  MOE_REQUIRE(router == 2 || softmax_dtype == MESH_MOE_F32, MESH_MOE_E_ARG,
              "router_summaries: only the ntlb router runs its softmax in "
              "bfloat16");
  SummaryParams p;
  p.G = G; p.S = S; p.E = E; p.K = k; p.router = router;
  p.tt = summary_tokens_per_block(E);
  p.nblk = (S + p.tt - 1) / p.tt;
  const size_t lds = sizeof(float) * ((size_t)p.tt * (E + 1 + SUM_HEAD) + E);
  dim3 grid((unsigned)p.nblk, (unsigned)G);
  const bool imp_bf16 = importance != nullptr && importance_dtype == MESH_MOE_BF16;
#define MOE_SUMMARY(IT_, ST_)                                                 \
  do {                                                                        \
    auto kfn = router_summary_kernel<IT_, ST_>;                               \
    MOE_ALLOW_LDS(kfn, lds);                                                  \
    kfn<<<grid, SUM_THREADS, lds, st>>>(p, logits, (const IT_*)importance,    \
                                        router == 1 ? kept : nullptr, ws);    \
  } while (0)
  if (softmax_dtype == MESH_MOE_BF16) {
    if (imp_bf16) MOE_SUMMARY(bf16_t, bf16_t); else MOE_SUMMARY(float, bf16_t);
  } else {
    if (imp_bf16) MOE_SUMMARY(bf16_t, float); else MOE_SUMMARY(float, float);
  }
#undef MOE_SUMMARY
  MOE_CHECK_LAUNCH("router_summaries");
  router_summary_finish_kernel<<<1, SUM_FINISH_THREADS,
                                 sizeof(float) * (SUM_HEAD + E), st>>>(
      p, ws, num_microbatches, out);
  MOE_CHECK_LAUNCH("router_summaries (finish)");
  return 0;
}
