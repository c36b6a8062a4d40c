// Expert-selection ("expert choice") gating for gfx950: every expert picks, per
// group, the `capacity` tokens it likes best
// (mesh_tensorflow/transformer/moe.py:1057-1173, _expert_selection_gating).
//
// A token can sit in the slots of several experts or of none, so the routing
// record is per SLOT, not per token:
//   slot_token  [G,E,C] int32   token (index within the group) of each slot
//   slot_weight [G,E,C] float32 combine weight of that slot
//   tok_slot    [G,S,E] int16   slot the token holds at expert e, -1 if none
// and the dispatch / combine einsums (moe.py:443-447, :509-510) become a gather
// per slot and a sum over the (at most E) slots of a token.
#include "common.h"

namespace mesh_moe {

struct ChoiceParams {
  int G, S, E, C;
  int normalize;  // divide by the number of experts that chose the token
  int num_microbatches;
};

__global__ void choice_clear_kernel(int32_t* num_routed, int64_t n_tok,
                                    int16_t* tok_slot, int64_t n_ts) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_ts;
       i += stride) {
    tok_slot[i] = (int16_t)-1;
    if (i < n_tok) num_routed[i] = 0;
  }
}

__device__ __forceinline__ float block_reduce(float v, float* red, bool is_max) {
  // 256 threads = 4 wavefronts
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
  for (int w = 1; w < 4; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

// One block per (expert, group): softmax over the group's tokens
// (moe.py:1094-1098; tokens with importance 0 get -1e9 first), then the C
// largest probabilities in descending order, equal ones in token order (the
// order of tf.math.top_k, ops.py:4934-4942): rank = number of tokens that beat
// this one.
template <typename IT>
__global__ __launch_bounds__(256) void choice_select_kernel(
    ChoiceParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, int32_t* __restrict__ slot_token,
    float* __restrict__ slot_prob, int16_t* __restrict__ tok_slot,
    int32_t* __restrict__ num_routed, float* __restrict__ lse_out,
    bool by_threshold) {
  extern __shared__ float pr[];  // [S] + 4 (+ 8 + 2 C with by_threshold)
  float* red = pr + p.S;
  const int e = blockIdx.x, g = blockIdx.y;
  const int S = p.S, E = p.E, C = p.C;
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)g * S;
  float m = -INFINITY;
  for (int s = tid; s < S; s += 256) {
    float x = logits[(base + s) * E + e];
    if (importance != nullptr && load_f32<IT>(importance + base + s) == 0.0f)
      x = x + (-1e9f);
    pr[s] = x;
    m = fmaxf(m, x);
  }
  m = block_reduce(m, red, true);
  const float negm = -m;
  float sum = 0.f;
  for (int s = tid; s < S; s += 256) sum += expf(pr[s] + negm);
  sum = block_reduce(sum, red, false);
  const float lse = logf(sum) + m;
  const float neglse = -lse;
  __syncthreads();
  for (int s = tid; s < S; s += 256) pr[s] = expf(pr[s] + neglse);
  if (tid == 0) lse_out[(int64_t)g * E + e] = lse;
  __syncthreads();
  auto emit = [&](int s, int rank, float ps) {
    const int64_t slot = ((int64_t)g * E + e) * C + rank;
    slot_token[slot] = s;
    slot_prob[slot] = ps;
    tok_slot[(base + s) * E + e] = (int16_t)rank;
    atomicAdd(num_routed + base + s, 1);
  };
  if (!by_threshold) {
    // every token against every token
    for (int s = tid; s < S; s += 256) {
      const float ps = pr[s];
      int rank = 0;
      for (int s2 = 0; s2 < S; ++s2) {
        const float p2 = pr[s2];
        rank += (p2 > ps || (p2 == ps && s2 < s)) ? 1 : 0;
      }
      if (rank < C) emit(s, rank, ps);
    }
    return;
  }
  // The C-th largest probability first (probabilities are >= 0, so their bit
  // patterns order like unsigned integers): the largest T with at least C
  // tokens >= T, found bit by bit.  Tokens above T (fewer than C) are ranked
  // among themselves; tokens equal to T follow in token order.
  int* iscr = reinterpret_cast<int*>(red + 4);          // [8]
  uint32_t* key_a = reinterpret_cast<uint32_t*>(iscr + 8);  // [C]
  int* tok_a = reinterpret_cast<int*>(key_a + C);       // [C]
  const uint32_t* key = reinterpret_cast<const uint32_t*>(pr);
  const int lane = tid & 63, wave = tid >> 6;
  // thread tid owns tokens [s_lo, s_hi): contiguous, so that compaction keeps
  // the token order
  const int per = (S + 255) / 256;
  const int s_lo = min(S, tid * per), s_hi = min(S, s_lo + per);
  auto block_count = [&](int v) {       // sum over the block, to every thread
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if (lane == 0) iscr[wave] = v;
    __syncthreads();
    return iscr[0] + iscr[1] + iscr[2] + iscr[3];
  };
  uint32_t thr = 0u;
  for (int bit = 30; bit >= 0; --bit) {
    const uint32_t trial = thr | (1u << bit);
    int cnt = 0;
    for (int s = s_lo; s < s_hi; ++s) cnt += key[s] >= trial ? 1 : 0;
    if (block_count(cnt) >= C) thr = trial;
  }
  // exclusive positions of this thread's tokens among those above / equal
  int n_gt = 0, n_eq = 0;
  for (int s = s_lo; s < s_hi; ++s) {
    n_gt += key[s] > thr ? 1 : 0;
    n_eq += key[s] == thr ? 1 : 0;
  }
  auto block_scan = [&](int v, int* total) {   // exclusive prefix over threads
    int inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int o = __shfl_up(inc, off, 64);
      if (lane >= off) inc += o;
    }
    __syncthreads();
    if (lane == 63) iscr[4 + wave] = inc;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += iscr[4 + w];
    *total = iscr[4] + iscr[5] + iscr[6] + iscr[7];
    return before + inc - v;
  };
  int total_gt, total_eq;
  int at_gt = block_scan(n_gt, &total_gt);
  int at_eq = block_scan(n_eq, &total_eq);
  for (int s = s_lo; s < s_hi; ++s) {
    const uint32_t k = key[s];
    if (k > thr) {
      key_a[at_gt] = k;
      tok_a[at_gt] = s;
      ++at_gt;
    } else if (k == thr) {
      const int rank = total_gt + at_eq;
      ++at_eq;
      if (rank < C) emit(s, rank, pr[s]);
    }
  }
  __syncthreads();
  for (int a = tid; a < total_gt; a += 256) {
    const uint32_t k = key_a[a];
    int rank = 0;
    // (the list is in token order: equal keys before position a come first)
    for (int b2 = 0; b2 < total_gt; ++b2) {
      const uint32_t k2 = key_a[b2];
      rank += (k2 > k || (k2 == k && b2 < a)) ? 1 : 0;
    }
    emit(tok_a[a], rank, __uint_as_float(k));
  }
}

// One block per (group, chunk of 256 tokens), one thread per token: combine
// weights (probability over the number of experts that chose the token,
// moe.py:1119-1123) and the chunk's share of the group's loss term
// mean(agg^2 * sum_s importance) * S with agg = mean_e p * (importance == 1)
// (moe.py:1125-1147): part[g][chunk] = (sum agg^2, sum importance).
template <typename IT>
__global__ __launch_bounds__(256) void choice_finish_kernel(
    ChoiceParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, const float* __restrict__ lse,
    const float* __restrict__ slot_prob, const int16_t* __restrict__ tok_slot,
    const int32_t* __restrict__ num_routed, float* __restrict__ slot_weight,
    float2* __restrict__ part) {
  extern __shared__ float fin_smem[];   // lse of the group [E], then 4
  float* lse_s = fin_smem;
  float* red = fin_smem + p.E;
  const int g = blockIdx.y, chunk = blockIdx.x;
  const int S = p.S, E = p.E, C = p.C;
  const int64_t base = (int64_t)g * S;
  const float inv_e = (float)(1.0 / (double)E);
  for (int e = threadIdx.x; e < E; e += 256) lse_s[e] = lse[(int64_t)g * E + e];
  __syncthreads();
  float sq = 0.f, imp_sum = 0.f;
  const int s = chunk * 256 + threadIdx.x;
  if (s < S) {
    const int64_t t = base + s;
    float imp = 1.0f;
    if (importance != nullptr) imp = load_f32<IT>(importance + t);
    const float mask = imp == 0.0f ? -1e9f : 0.0f;
    const float recip =
        p.normalize ? 1.0f / fmaxf((float)num_routed[t], 1.0f) : 1.0f;
    float agg = 0.f;
    for (int e = 0; e < E; ++e) {
      float x = logits[t * E + e];
      if (imp == 0.0f) x = x + mask;
      agg += expf(x + (-lse_s[e]));
      const int c = tok_slot[t * E + e];
      if (c >= 0) {
        const int64_t slot = ((int64_t)g * E + e) * C + c;
        slot_weight[slot] = slot_prob[slot] * recip;
      }
    }
    agg = (agg * inv_e) * (imp == 1.0f ? 1.0f : 0.0f);
    sq = agg * agg;
    imp_sum = imp;
  }
  sq = block_reduce(sq, red, false);
  imp_sum = block_reduce(imp_sum, red, false);
  if (threadIdx.x == 0)
    part[(int64_t)g * gridDim.x + chunk] = make_float2(sq, imp_sum);
}

// The loss from the chunks' shares, summed in chunk order (one thread per
// group), then in group order.
__global__ __launch_bounds__(256) void choice_loss_kernel(
    ChoiceParams p, const float2* __restrict__ part, int chunks,
    float* __restrict__ loss) {
  __shared__ float term[256];
  float s = 0.f;
  for (int g0 = 0; g0 < p.G; g0 += 256) {
    const int g = g0 + threadIdx.x;
    float sq = 0.f, imp = 0.f;
    if (g < p.G) {
      for (int c = 0; c < chunks; ++c) {
        const float2 v = part[(int64_t)g * chunks + c];
        sq += v.x;
        imp += v.y;
      }
    }
    __syncthreads();
    term[threadIdx.x] = sq * imp;
    __syncthreads();
    if (threadIdx.x == 0) {
      const int n = min(256, p.G - g0);
      for (int i = 0; i < n; ++i) s += term[i];
    }
  }
  if (threadIdx.x != 0) return;
  float l = (s * (float)(1.0 / ((double)p.G * (double)p.S))) * (float)p.S;
  if (p.num_microbatches > 1)
    l = l * (float)(1.0 / (double)p.num_microbatches);
  loss[0] = l;
}

constexpr int CH_ROWS = 4;  // wavefronts (rows) per block

// expert_in[e,g,c,:] = x[g, slot_token[g,e,c], :]
template <typename T>
__global__ __launch_bounds__(256) void slot_dispatch_kernel(
    const T* __restrict__ x, const int32_t* __restrict__ slot_token,
    T* __restrict__ expert_in, int G, int S, int E, int C, int M,
    int64_t n_slots, bool vec) {
  const int lane = threadIdx.x & 63;
  const int64_t j = (int64_t)blockIdx.x * CH_ROWS + (threadIdx.x >> 6);
  if (j >= n_slots) return;
  // j enumerates the destination [E,G,C]
  const int c = (int)(j % C);
  const int g = (int)((j / C) % G);
  const int e = (int)(j / ((int64_t)C * G));
  const int s = slot_token[((int64_t)g * E + e) * C + c];
  const T* src = x + ((int64_t)g * S + s) * M;
  T* dst = expert_in + j * M;
  if (vec) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    const int nv = M / (16 / (int)sizeof(T));
    for (int i = lane; i < nv; i += 64) store_streaming(d4 + i, s4[i]);
  } else {
    for (int i = lane; i < M; i += 64) dst[i] = src[i];
  }
}

// out[g,s,:] = sum_e w * y[e,g,tok_slot[g,s,e],:] over the experts that chose
// the token, float32 accumulate in expert order, one rounding.  One wavefront
// per token: the experts that chose it are found once (a ballot over 64 experts
// at a time) and listed in LDS with their row and weight; the rows are then
// read with 16-byte loads, 512 / 256 columns of all listed rows at a time.
constexpr int SC_MAX_E = 512;

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void slot_combine_kernel(
    const T* __restrict__ y, const int16_t* __restrict__ tok_slot,
    const float* __restrict__ slot_weight, T* __restrict__ out, int G, int S,
    int E, int C, int N, int64_t T_tokens) {
  constexpr int VN = Vec16B<T>::N;
  __shared__ int64_t rows[CH_ROWS][SC_MAX_E];
  __shared__ float wts[CH_ROWS][SC_MAX_E];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * CH_ROWS + wave;
  if (t >= T_tokens) return;
  const int g = (int)(t / S);
  const int16_t* ts = tok_slot + t * E;
  int n = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    const int c = e < E ? (int)ts[e] : -1;
    const unsigned long long m = __ballot(c >= 0);
    if (c >= 0) {
      const int at = n + __popcll(m & ((1ull << lane) - 1ull));
      rows[wave][at] = (((int64_t)e * G + g) * C + c) * N;
      wts[wave][at] = round_to<T>(slot_weight[((int64_t)g * E + e) * C + c]);
    }
    n += __popcll(m);
  }
  // (the list is written and read by the same wavefront: LDS operations of a
  // wavefront complete in order)
  T* dst = out + t * N;
  if (VEC) {
    for (int i0 = lane * VN; i0 < N; i0 += 64 * VN) {
      float acc[VN];
#pragma unroll
      for (int j = 0; j < VN; ++j) acc[j] = 0.f;
      for (int k = 0; k < n; ++k) {
        float v[VN];
        unpack16(load_streaming(reinterpret_cast<const uint4*>(
                     y + rows[wave][k] + i0)), v, T());
        const float w = wts[wave][k];
#pragma unroll
        for (int j = 0; j < VN; ++j) acc[j] += w * v[j];
      }
      store_streaming(reinterpret_cast<uint4*>(dst + i0), pack16(acc, T()));
    }
  } else {
    for (int i = lane; i < N; i += 64) {
      float acc = 0.f;
      for (int k = 0; k < n; ++k)
        acc += wts[wave][k] * load_f32<T>(y + rows[wave][k] + i);
      store_f32<T>(dst + i, acc);
    }
  }
}

// ---------------------------------------------------------------------------
// Backward.
// ---------------------------------------------------------------------------

// dy[e,g,c,:] = w * dout[g, slot_token[g,e,c], :] (w = the slot's combine weight
// as the activation dtype holds it), dweight[g,e,c] = <dout[g,token,:],
// y[e,g,c,:]> in float32.  One wavefront per slot.
template <typename T>
__global__ __launch_bounds__(256) void slot_combine_backward_kernel(
    const T* __restrict__ dout, const T* __restrict__ y,
    const int32_t* __restrict__ slot_token,
    const float* __restrict__ slot_weight, T* __restrict__ dy,
    float* __restrict__ dweight, int G, int S, int E, int C, int N,
    int64_t n_slots, bool vec) {
  const int lane = threadIdx.x & 63;
  const int64_t j = (int64_t)blockIdx.x * CH_ROWS + (threadIdx.x >> 6);
  if (j >= n_slots) return;
  // j enumerates [E,G,C] (the layout of y and dy)
  const int c = (int)(j % C);
  const int g = (int)((j / C) % G);
  const int e = (int)(j / ((int64_t)C * G));
  const int64_t slot = ((int64_t)g * E + e) * C + c;
  const float w = round_to<T>(slot_weight[slot]);
  const T* drow = dout + ((int64_t)g * S + slot_token[slot]) * N;
  const T* yrow = y + j * N;
  T* dst = dy + j * N;
  float dot = 0.f;
  if (vec) {
    // 16-byte pieces, the loads of a batch of eight all issued before the
    // first use
    constexpr int VN = Vec16B<T>::N;
    constexpr int UN = 8;
    const int nv = N / VN;
    const uint4* d4 = reinterpret_cast<const uint4*>(drow);
    const uint4* y4 = reinterpret_cast<const uint4*>(yrow);
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int base = lane; base < nv; base += 64 * UN) {
      uint4 dr[UN], yr[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        dr[u] = i < nv ? load_streaming(d4 + i) : z;
        yr[u] = i < nv ? load_streaming(y4 + i) : z;
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int i = base + u * 64;
        if (i >= nv) continue;
        float d[VN], yv[VN], o[VN];
        unpack16(dr[u], d, T());
        unpack16(yr[u], yv, T());
#pragma unroll
        for (int q = 0; q < VN; ++q) {
          dot += d[q] * yv[q];
          o[q] = w * d[q];
        }
        store_streaming(reinterpret_cast<uint4*>(dst) + i, pack16(o, T()));
      }
    }
  } else {
    for (int i = lane; i < N; i += 64) {
      const float d = load_f32<T>(drow + i);
      dot += d * load_f32<T>(yrow + i);
      store_f32<T>(dst + i, w * d);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
  if (lane == 0) dweight[slot] = dot;
}

// dx[g,s,:] = sum over the experts that chose the token of dexpert_in[e,g,c,:]
// (+ dlogits[g,s,:] . w_gate^T when the router's share is wanted), float32
// accumulate in expert order, one rounding.  One wavefront per token.
template <typename T>
__global__ __launch_bounds__(256) void slot_dispatch_backward_kernel(
    const T* __restrict__ dxe, const int16_t* __restrict__ tok_slot,
    const float* __restrict__ dlogits, const T* __restrict__ wgp,
    T* __restrict__ dx, int G, int S, int E, int C, int M, int64_t T_tokens) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * CH_ROWS + (threadIdx.x >> 6);
  if (t >= T_tokens) return;
  const int g = (int)(t / S);
  const int16_t* ts = tok_slot + t * E;
  const float* dl = dlogits ? dlogits + t * E : nullptr;
  T* dst = dx + t * M;
  for (int i0 = 0; i0 < M; i0 += 64 * 4) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int e = 0; e < E; ++e) {
      const int c = ts[e];
      if (c >= 0) {
        const T* row = dxe + (((int64_t)e * G + g) * C + c) * M;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 64 + lane;
          if (i < M) acc[u] += load_f32<T>(row + i);
        }
      }
    }
    if (dl != nullptr) {
      for (int e = 0; e < E; ++e) {
        const float d = dl[e];
        const T* row = wgp + (int64_t)e * M;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 64 + lane;
          if (i < M) acc[u] = fmaf(d, load_f32<T>(row + i), acc[u]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * 64 + lane;
      if (i < M) store_f32<T>(dst + i, acc[u]);
    }
  }
}

// log-sum-exp over the group's tokens of every (group, expert) column, as the
// forward pass computes it.  One block per (expert, group).
template <typename IT>
__global__ __launch_bounds__(256) void choice_lse_kernel(
    ChoiceParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, float* __restrict__ lse_out) {
  __shared__ float red[4];
  const int e = blockIdx.x, g = blockIdx.y;
  const int S = p.S, E = p.E;
  const int64_t base = (int64_t)g * S;
  auto value = [&](int s) {
    float x = logits[(base + s) * E + e];
    if (importance != nullptr && load_f32<IT>(importance + base + s) == 0.0f)
      x = x + (-1e9f);
    return x;
  };
  float m = -INFINITY;
  for (int s = threadIdx.x; s < S; s += 256) m = fmaxf(m, value(s));
  m = block_reduce(m, red, true);
  const float negm = -m;
  float sum = 0.f;
  for (int s = threadIdx.x; s < S; s += 256) sum += expf(value(s) + negm);
  sum = block_reduce(sum, red, false);
  if (threadIdx.x == 0) lse_out[(int64_t)g * E + e] = logf(sum) + m;
}

// One block per group: per token 1 / max(#experts that chose it, 1) and the
// loss's share of d(p[g,s,e]) (the same for every e):
// d_loss * 2 * agg * sum_s(importance) * (importance == 1) / (E * G * mb).
template <typename IT>
__global__ __launch_bounds__(256) void choice_backward_token_kernel(
    ChoiceParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, const float* __restrict__ lse,
    const int16_t* __restrict__ tok_slot, const float* __restrict__ d_loss,
    float loss_scale, float* __restrict__ recip_out,
    float* __restrict__ dloss_out) {
  __shared__ float red[4];
  const int g = blockIdx.x;
  const int S = p.S, E = p.E;
  const int64_t base = (int64_t)g * S;
  const float inv_e = (float)(1.0 / (double)E);
  float imp_sum = 0.f;
  for (int s = threadIdx.x; s < S; s += 256)
    imp_sum += importance != nullptr ? load_f32<IT>(importance + base + s) : 1.0f;
  imp_sum = block_reduce(imp_sum, red, false);
  const float mb =
      p.num_microbatches > 1 ? (float)(1.0 / (double)p.num_microbatches) : 1.0f;
  const float coef = d_loss[0] * loss_scale * mb * (float)(2.0 / (double)p.G) *
                     imp_sum * inv_e;
  for (int s = threadIdx.x; s < S; s += 256) {
    const int64_t t = base + s;
    float imp = 1.0f;
    if (importance != nullptr) imp = load_f32<IT>(importance + t);
    float agg = 0.f;
    int routed = 0;
    for (int e = 0; e < E; ++e) {
      float x = logits[t * E + e];
      if (imp == 0.0f) x = x + (-1e9f);
      agg += expf(x + (-lse[(int64_t)g * E + e]));
      routed += tok_slot[t * E + e] >= 0 ? 1 : 0;
    }
    const float is_one = imp == 1.0f ? 1.0f : 0.0f;
    agg = (agg * inv_e) * is_one;
    recip_out[t] = p.normalize ? 1.0f / fmaxf((float)routed, 1.0f) : 1.0f;
    dloss_out[t] = coef * agg * is_one;
  }
}

// One block per (expert, group): d(logits[g,:,e]) = p * (dp - sum_s p * dp),
// dp = dweight[slot] / #experts of the token (chosen tokens) + the loss's share.
template <typename IT>
__global__ __launch_bounds__(256) void choice_backward_column_kernel(
    ChoiceParams p, const float* __restrict__ logits,
    const IT* __restrict__ importance, const float* __restrict__ lse,
    const int16_t* __restrict__ tok_slot, const float* __restrict__ dweight,
    const float* __restrict__ recip, const float* __restrict__ dloss_tok,
    float* __restrict__ dlogits) {
  __shared__ float red[4];
  const int e = blockIdx.x, g = blockIdx.y;
  const int S = p.S, E = p.E, C = p.C;
  const int64_t base = (int64_t)g * S;
  const float neglse = -lse[(int64_t)g * E + e];
  auto prob_and_dp = [&](int s, float& dp) {
    const int64_t t = base + s;
    float x = logits[t * E + e];
    if (importance != nullptr && load_f32<IT>(importance + t) == 0.0f)
      x = x + (-1e9f);
    dp = dloss_tok[t];
    const int c = tok_slot[t * E + e];
    if (c >= 0) dp += dweight[((int64_t)g * E + e) * C + c] * recip[t];
    return expf(x + neglse);
  };
  float inner = 0.f;
  for (int s = threadIdx.x; s < S; s += 256) {
    float dp;
    const float ps = prob_and_dp(s, dp);
    inner += ps * dp;
  }
  inner = block_reduce(inner, red, false);
  for (int s = threadIdx.x; s < S; s += 256) {
    float dp;
    const float ps = prob_and_dp(s, dp);
    dlogits[(base + s) * E + e] = ps * (dp - inner);
  }
}

}  // namespace mesh_moe

using namespace mesh_moe;

extern "C" size_t mesh_moe_expert_choice_workspace_bytes(int G, int S, int E,
                                                         int C) {
  if (G < 1 || S < 1 || E < 1 || C < 1) return 0;
  return sizeof(int32_t) * (size_t)G * S + sizeof(float) * (size_t)G * E +
         sizeof(float) * (size_t)G * E * C +
         sizeof(float) * 2 * (size_t)G * (((size_t)S + 255) / 256) + 4 * 256;
}

extern "C" int mesh_moe_expert_choice_gating(
    const float* logits, const void* importance, int importance_dtype, int G,
    int S, int E, int C, int normalize, int num_microbatches,
    int32_t* slot_token, float* slot_weight, int16_t* tok_slot, float* loss,
    void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && slot_token && slot_weight && tok_slot && loss &&
                  workspace, MESH_MOE_E_ARG,
              "expert_choice_gating: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1, MESH_MOE_E_ARG,
              "expert_choice_gating: bad sizes G=%d S=%d E=%d C=%d", G, S, E,
              C);
  MOE_REQUIRE(C <= S, MESH_MOE_E_ARG,
              "expert_choice_gating: capacity %d > group size %d", C, S);
  MOE_REQUIRE(S <= 32768 && E <= 65535 && G <= 65535, MESH_MOE_E_UNSUPPORTED,
              "expert_choice_gating: S=%d > 32768 or E, G > 65535", S);
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "expert_choice_gating: bad importance dtype %d",
              importance_dtype);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_expert_choice_workspace_bytes(G, S, E, C),
              MESH_MOE_E_ARG, "expert_choice_gating: workspace too small");
  ChoiceParams p;
  p.G = G; p.S = S; p.E = E; p.C = C;
  p.normalize = normalize ? 1 : 0;
  p.num_microbatches = num_microbatches;
  auto up = [](uintptr_t v) { return (v + 255) & ~(uintptr_t)255; };
  int32_t* num_routed = (int32_t*)up((uintptr_t)workspace);
  float* lse = (float*)up((uintptr_t)(num_routed + (size_t)G * S));
  float* slot_prob = (float*)up((uintptr_t)(lse + (size_t)G * E));
  float* gsum = (float*)up((uintptr_t)(slot_prob + (size_t)G * E * C));
  hipStream_t st = (hipStream_t)stream;
  const int64_t n_tok = (int64_t)G * S, n_ts = n_tok * E;
  const unsigned cb = (unsigned)((n_ts + 255) / 256 < 8192 ? (n_ts + 255) / 256
                                                            : 8192);
  choice_clear_kernel<<<cb, 256, 0, st>>>(num_routed, n_tok, tok_slot, n_ts);
  MOE_CHECK_LAUNCH("expert_choice_gating (clear)");
  // the threshold form needs two lists of C entries next to the probabilities
  const size_t smem_thr = sizeof(float) * ((size_t)S + 4 + 8 + 2 * (size_t)C);
  const bool by_threshold = smem_thr <= 150 * 1024;
  const size_t smem = by_threshold ? smem_thr : sizeof(float) * ((size_t)S + 4);
  dim3 grid((unsigned)E, (unsigned)G);
  const bool bf = importance && importance_dtype == MESH_MOE_BF16;
  if (bf) {
    auto k = choice_select_kernel<bf16_t>;
    MOE_ALLOW_LDS(k, smem);
    k<<<grid, 256, smem, st>>>(p, logits, (const bf16_t*)importance, slot_token,
                               slot_prob, tok_slot, num_routed, lse,
                               by_threshold);
  } else {
    auto k = choice_select_kernel<float>;
    MOE_ALLOW_LDS(k, smem);
    k<<<grid, 256, smem, st>>>(p, logits, (const float*)importance, slot_token,
                               slot_prob, tok_slot, num_routed, lse,
                               by_threshold);
  }
  MOE_CHECK_LAUNCH("expert_choice_gating (select)");
  const int chunks = (S + 255) / 256;
  const dim3 fgrid((unsigned)chunks, (unsigned)G);
  const size_t fsmem = sizeof(float) * ((size_t)E + 4);
  float2* part = reinterpret_cast<float2*>(gsum);
  if (bf)
    choice_finish_kernel<bf16_t><<<fgrid, 256, fsmem, st>>>(
        p, logits, (const bf16_t*)importance, lse, slot_prob, tok_slot,
        num_routed, slot_weight, part);
  else
    choice_finish_kernel<float><<<fgrid, 256, fsmem, st>>>(
        p, logits, (const float*)importance, lse, slot_prob, tok_slot,
        num_routed, slot_weight, part);
  MOE_CHECK_LAUNCH("expert_choice_gating (finish)");
  choice_loss_kernel<<<1, 256, 0, st>>>(p, part, chunks, loss);
  MOE_CHECK_LAUNCH("expert_choice_gating (loss)");
  return 0;
}

extern "C" int mesh_moe_slot_dispatch(const void* x, const int32_t* slot_token,
                                      void* expert_in, int G, int S, int E,
                                      int C, int M, int dtype, void* stream) {
  MOE_REQUIRE(x && slot_token && expert_in, MESH_MOE_E_ARG,
              "slot_dispatch: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "slot_dispatch: bad dtype %d",
              dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1, MESH_MOE_E_ARG,
              "slot_dispatch: bad sizes G=%d S=%d E=%d C=%d M=%d", G, S, E, C,
              M);
  const int64_t n_slots = (int64_t)G * E * C;
  const int64_t nblocks = (n_slots + CH_ROWS - 1) / CH_ROWS;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "slot_dispatch: too many slots (%lld)", (long long)n_slots);
  const bool vec = ((size_t)M * dtype_size(dtype)) % 16 == 0 &&
                   ((uintptr_t)x & 15) == 0 && ((uintptr_t)expert_in & 15) == 0;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32)
    slot_dispatch_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)x, slot_token, (float*)expert_in, G, S, E, C, M, n_slots,
        vec);
  else
    slot_dispatch_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)x, slot_token, (bf16_t*)expert_in, G, S, E, C, M,
        n_slots, vec);
  MOE_CHECK_LAUNCH("slot_dispatch");
  return 0;
}

extern "C" int mesh_moe_slot_combine(const void* y, const int16_t* tok_slot,
                                     const float* slot_weight, void* out,
                                     int G, int S, int E, int C, int N,
                                     int dtype, void* stream) {
  MOE_REQUIRE(y && tok_slot && slot_weight && out, MESH_MOE_E_ARG,
              "slot_combine: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "slot_combine: bad dtype %d",
              dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && N >= 1, MESH_MOE_E_ARG,
              "slot_combine: bad sizes G=%d S=%d E=%d C=%d N=%d", G, S, E, C,
              N);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t nblocks = (T_tokens + CH_ROWS - 1) / CH_ROWS;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "slot_combine: too many rows (%lld)", (long long)T_tokens);
  hipStream_t st = (hipStream_t)stream;
  MOE_REQUIRE(E <= SC_MAX_E, MESH_MOE_E_UNSUPPORTED,
              "slot_combine: E=%d > %d", E, SC_MAX_E);
  const bool vec = ((size_t)N * dtype_size(dtype)) % 16 == 0 &&
                   (((uintptr_t)y | (uintptr_t)out) % 16) == 0;
#define MOE_SLOT_COMBINE(T, V)                                              \
  slot_combine_kernel<T, V><<<(unsigned)nblocks, 256, 0, st>>>(             \
      (const T*)y, tok_slot, slot_weight, (T*)out, G, S, E, C, N, T_tokens)
  if (dtype == MESH_MOE_F32) {
    if (vec) MOE_SLOT_COMBINE(float, true); else MOE_SLOT_COMBINE(float, false);
  } else {
    if (vec) MOE_SLOT_COMBINE(bf16_t, true); else MOE_SLOT_COMBINE(bf16_t, false);
  }
#undef MOE_SLOT_COMBINE
  MOE_CHECK_LAUNCH("slot_combine");
  return 0;
}

extern "C" int mesh_moe_slot_combine_backward(
    const void* dout, const void* y, const int32_t* slot_token,
    const float* slot_weight, void* dy, float* dweight, int G, int S, int E,
    int C, int N, int dtype, void* stream) {
  MOE_REQUIRE(dout && y && slot_token && slot_weight && dy && dweight,
              MESH_MOE_E_ARG, "slot_combine_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "slot_combine_backward: bad dtype %d", dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && N >= 1, MESH_MOE_E_ARG,
              "slot_combine_backward: bad sizes G=%d S=%d E=%d C=%d N=%d", G, S,
              E, C, N);
  const int64_t n_slots = (int64_t)G * E * C;
  const int64_t nblocks = (n_slots + CH_ROWS - 1) / CH_ROWS;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "slot_combine_backward: too many slots (%lld)",
              (long long)n_slots);
  const bool vec = ((size_t)N * dtype_size(dtype)) % 16 == 0 &&
                   (((uintptr_t)dout | (uintptr_t)y | (uintptr_t)dy) & 15) == 0;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32)
    slot_combine_backward_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)dout, (const float*)y, slot_token, slot_weight,
        (float*)dy, dweight, G, S, E, C, N, n_slots, vec);
  else
    slot_combine_backward_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)dout, (const bf16_t*)y, slot_token, slot_weight,
        (bf16_t*)dy, dweight, G, S, E, C, N, n_slots, vec);
  MOE_CHECK_LAUNCH("slot_combine_backward");
  return 0;
}

namespace mesh_moe {
bool launch_slot_dispatch_backward_mfma(
    const void* dexpert_in, const int16_t* tok_slot, const float* dlogits,
    const void* w_gate, void* dx, int G, int S, int E, int C, int M, int dtype,
    hipStream_t st, int* rc);
}

extern "C" int mesh_moe_slot_dispatch_backward(
    const void* dexpert_in, const int16_t* tok_slot, const float* dlogits,
    const void* w_gate_packed, const void* w_gate, void* dx, int G, int S,
    int E, int C, int M, int dtype, void* stream) {
  MOE_REQUIRE(dexpert_in && tok_slot && dx, MESH_MOE_E_ARG,
              "slot_dispatch_backward: null pointer");
  MOE_REQUIRE((dlogits == nullptr) == (w_gate_packed == nullptr),
              MESH_MOE_E_ARG,
              "slot_dispatch_backward: dlogits and w_gate_packed go together");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "slot_dispatch_backward: bad dtype %d", dtype);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1, MESH_MOE_E_ARG,
              "slot_dispatch_backward: bad sizes G=%d S=%d E=%d C=%d M=%d", G,
              S, E, C, M);
  const int64_t T_tokens = (int64_t)G * S;
  const int64_t nblocks = (T_tokens + CH_ROWS - 1) / CH_ROWS;
  MOE_REQUIRE(nblocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "slot_dispatch_backward: too many rows (%lld)",
              (long long)T_tokens);
  hipStream_t st = (hipStream_t)stream;
  int rc = 0;
  if (launch_slot_dispatch_backward_mfma(dexpert_in, tok_slot, dlogits, w_gate,
                                         dx, G, S, E, C, M, dtype, st, &rc))
    return rc;
  if (dtype == MESH_MOE_F32)
    slot_dispatch_backward_kernel<float><<<(unsigned)nblocks, 256, 0, st>>>(
        (const float*)dexpert_in, tok_slot, dlogits,
        (const float*)w_gate_packed, (float*)dx, G, S, E, C, M, T_tokens);
  else
    slot_dispatch_backward_kernel<bf16_t><<<(unsigned)nblocks, 256, 0, st>>>(
        (const bf16_t*)dexpert_in, tok_slot, dlogits,
        (const bf16_t*)w_gate_packed, (bf16_t*)dx, G, S, E, C, M, T_tokens);
  MOE_CHECK_LAUNCH("slot_dispatch_backward");
  return 0;
}

extern "C" size_t mesh_moe_expert_choice_backward_workspace_bytes(int G, int S,
                                                                  int E) {
  if (G < 1 || S < 1 || E < 1) return 0;
  return sizeof(float) * ((size_t)G * E + 2 * (size_t)G * S) + 3 * 256;
}

extern "C" int mesh_moe_expert_choice_backward(
    const float* logits, const void* importance, int importance_dtype,
    const int16_t* tok_slot, const float* dweight, const float* d_loss,
    double loss_scale, int G, int S, int E, int C, int normalize,
    int num_microbatches, float* dlogits, void* workspace,
    size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(logits && tok_slot && dweight && d_loss && dlogits && workspace,
              MESH_MOE_E_ARG, "expert_choice_backward: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && C <= S, MESH_MOE_E_ARG,
              "expert_choice_backward: bad sizes G=%d S=%d E=%d C=%d", G, S, E,
              C);
  MOE_REQUIRE(E <= 65535 && G <= 65535, MESH_MOE_E_UNSUPPORTED,
              "expert_choice_backward: E or G > 65535");
  MOE_REQUIRE(!importance || valid_dtype(importance_dtype), MESH_MOE_E_ARG,
              "expert_choice_backward: bad importance dtype %d",
              importance_dtype);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_expert_choice_backward_workspace_bytes(G, S, E),
              MESH_MOE_E_ARG, "expert_choice_backward: workspace too small");
  ChoiceParams p;
  p.G = G; p.S = S; p.E = E; p.C = C;
  p.normalize = normalize ? 1 : 0;
  p.num_microbatches = num_microbatches;
  auto up = [](uintptr_t v) { return (v + 255) & ~(uintptr_t)255; };
  float* lse = (float*)up((uintptr_t)workspace);
  float* recip = (float*)up((uintptr_t)(lse + (size_t)G * E));
  float* dloss_tok = (float*)up((uintptr_t)(recip + (size_t)G * S));
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)E, (unsigned)G);
  if (importance && importance_dtype == MESH_MOE_BF16) {
    const bf16_t* imp = (const bf16_t*)importance;
    choice_lse_kernel<bf16_t><<<grid, 256, 0, st>>>(p, logits, imp, lse);
    MOE_CHECK_LAUNCH("expert_choice_backward (lse)");
    choice_backward_token_kernel<bf16_t><<<G, 256, 0, st>>>(
        p, logits, imp, lse, tok_slot, d_loss, (float)loss_scale, recip,
        dloss_tok);
    MOE_CHECK_LAUNCH("expert_choice_backward (tokens)");
    choice_backward_column_kernel<bf16_t><<<grid, 256, 0, st>>>(
        p, logits, imp, lse, tok_slot, dweight, recip, dloss_tok, dlogits);
  } else {
    const float* imp = (const float*)importance;
    choice_lse_kernel<float><<<grid, 256, 0, st>>>(p, logits, imp, lse);
    MOE_CHECK_LAUNCH("expert_choice_backward (lse)");
    choice_backward_token_kernel<float><<<G, 256, 0, st>>>(
        p, logits, imp, lse, tok_slot, d_loss, (float)loss_scale, recip,
        dloss_tok);
    MOE_CHECK_LAUNCH("expert_choice_backward (tokens)");
    choice_backward_column_kernel<float><<<grid, 256, 0, st>>>(
        p, logits, imp, lse, tok_slot, dweight, recip, dloss_tok, dlogits);
  }
  MOE_CHECK_LAUNCH("expert_choice_backward (columns)");
  return 0;
}
