// The rest of a transformer block around the Mixture-of-Experts layer, for
// gfx950: RMS normalisation and multi-head self-attention.
//
// rms_norm follows sublayer_rms_norm, mesh_tensorflow/transformer/
// transformer.py:493-516: x * rsqrt(mean(square(x)) + epsilon) * scale, one
// rounding to the activation dtype per reference op, float32 accumulation.
//
// self_attention follows attention.attention, mesh_tensorflow/transformer/
// attention.py:27-88 with float32_logits (the default): logits = q . k in
// float32, plus a -1e9 bias where a key is not visible (attention.py:830-842),
// mtf.softmax in float32 (ops.py:5493-5541), weights cast to the activation
// dtype, outputs = weights . v.  The scaling 1/sqrt(d_kv) is folded into the
// query kernel's initialiser by the reference (attention.py:436-439), so none
// is applied here.
#include "common.h"

namespace mesh_moe {

// ---------------------------------------------------------------------------
// RMS norm: one wavefront per row.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_kernel(
    const T* __restrict__ x, const T* __restrict__ scale, T* __restrict__ y,
    int64_t rows, int M, float inv_m, float eps, bool vec16) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * M;
  T* yr = y + row * M;
  float sum = 0.f;
  if (sizeof(T) == 2 && vec16) {
    // bf16 rows in 16-byte pieces: 8 values per lane and step
    const uint4* xv = reinterpret_cast<const uint4*>(xr);
    const uint4* sv = reinterpret_cast<const uint4*>(scale);
    uint4* yv = reinterpret_cast<uint4*>(yr);
    const int chunks = M / 8;
    for (int c = lane; c < chunks; c += 64) {
      const uint4 p = xv[c];
      const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = __uint_as_float(w[j] << 16);
        const float b = __uint_as_float(w[j] & 0xffff0000u);
        sum += round_to<T>(a * a);
        sum += round_to<T>(b * b);
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    const float total = round_to<T>(sum);
    const float mean = round_to<T>(total * inv_m);
    const float var = round_to<T>(mean + eps);
    const float r = round_to<T>(1.0f / sqrtf(var));
    for (int c = lane; c < chunks; c += 64) {
      const uint4 p = xv[c], q = sv[c];
      const uint32_t w[4] = {p.x, p.y, p.z, p.w};
      const uint32_t g[4] = {q.x, q.y, q.z, q.w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = __uint_as_float(w[j] << 16);
        const float b = __uint_as_float(w[j] & 0xffff0000u);
        const float sa = __uint_as_float(g[j] << 16);
        const float sb = __uint_as_float(g[j] & 0xffff0000u);
        o[j] = f32x2_to_bf16x2(round_to<T>(a * r) * sa, round_to<T>(b * r) * sb);
      }
      yv[c] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    return;
  }
  for (int i = lane; i < M; i += 64) {
    const float v = load_f32<T>(xr + i);
    sum += round_to<T>(v * v);                              // mtf.square
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const float total = round_to<T>(sum);                     // reduce_sum
  const float mean = round_to<T>(total * inv_m);            // * (1 / M)
  const float var = round_to<T>(mean + eps);                // + epsilon
  const float r = round_to<T>(1.0f / sqrtf(var));           // rsqrt
  for (int i = lane; i < M; i += 64) {
    const float v = load_f32<T>(xr + i);
    const float s = load_f32<T>(scale + i);
    store_f32<T>(yr + i, round_to<T>(v * r) * s);
  }
}

// The same for bf16 rows of at most ITERS * 512 elements (16-byte aligned):
// the row stays in registers -- all its 16-byte loads are in flight together,
// and it is read once.
template <int ITERS>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ scale,
    bf16_t* __restrict__ y, int64_t rows, int M, float inv_m, float eps) {
  using T = bf16_t;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint4* xv = reinterpret_cast<const uint4*>(x + row * M);
  const uint4* sv = reinterpret_cast<const uint4*>(scale);
  uint4* yv = reinterpret_cast<uint4*>(y + row * M);
  const int chunks = M / 8;
  uint4 p[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + 64 * it;
    p[it] = c < chunks ? load_streaming(xv + c) : make_uint4(0, 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const uint32_t w[4] = {p[it].x, p[it].y, p[it].z, p[it].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a = __uint_as_float(w[j] << 16);
      const float b = __uint_as_float(w[j] & 0xffff0000u);
      sum += round_to<T>(a * a);
      sum += round_to<T>(b * b);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const float total = round_to<T>(sum);
  const float mean = round_to<T>(total * inv_m);
  const float var = round_to<T>(mean + eps);
  const float r = round_to<T>(1.0f / sqrtf(var));
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + 64 * it;
    if (c >= chunks) continue;
    const uint4 q = sv[c];
    const uint32_t w[4] = {p[it].x, p[it].y, p[it].z, p[it].w};
    const uint32_t g[4] = {q.x, q.y, q.z, q.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a = __uint_as_float(w[j] << 16);
      const float b = __uint_as_float(w[j] & 0xffff0000u);
      const float sa = __uint_as_float(g[j] << 16);
      const float sb = __uint_as_float(g[j] & 0xffff0000u);
      o[j] = f32x2_to_bf16x2(round_to<T>(a * r) * sa, round_to<T>(b * r) * sb);
    }
    store_streaming(yv + c, make_uint4(o[0], o[1], o[2], o[3]));
  }
}

// ---------------------------------------------------------------------------
// [B, L, H*D] -> [B*H, L, D]  (heads to the front)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void split_heads_kernel(const T* __restrict__ in, T* __restrict__ out,
                                   int B, int L, int H, int D) {
  const int64_t n = (int64_t)B * L * H * D;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const int d = (int)(i % D);
    int64_t r = i / D;
    const int l = (int)(r % L);
    r /= L;
    const int h = (int)(r % H);
    const int b = (int)(r / H);
    out[i] = in[(((int64_t)b * L + l) * H + h) * D + d];
  }
}

// [B*H, L, D] -> [B, L, H*D]
template <typename T>
__global__ void merge_heads_kernel(const T* __restrict__ in, T* __restrict__ out,
                                   int B, int L, int H, int D) {
  const int64_t n = (int64_t)B * L * H * D;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const int d = (int)(i % D);
    int64_t r = i / D;
    const int h = (int)(r % H);
    r /= H;
    const int l = (int)(r % L);
    const int b = (int)(r / L);
    out[i] = in[(((int64_t)b * H + h) * L + l) * D + d];
  }
}

// [B, L, H*D] -> [B*H, D, L]: the values as the K-contiguous second operand of
// weights . v.  32 x 32 tiles through LDS so both sides are coalesced.
template <typename T>
__global__ __launch_bounds__(256) void transpose_heads_kernel(
    const T* __restrict__ in, T* __restrict__ out, int B, int L, int H, int D) {
  __shared__ T tile[32][33];
  const int bh = blockIdx.z, b = bh / H, h = bh % H;
  const int l0 = blockIdx.x * 32, d0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
  for (int r = ty; r < 32; r += 8) {
    const int l = l0 + r, d = d0 + tx;
    if (l < L && d < D)
      tile[r][tx] = in[(((int64_t)b * L + l) * H + h) * D + d];
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int d = d0 + r, l = l0 + tx;
    if (l < L && d < D) out[((int64_t)bh * D + d) * L + l] = tile[tx][r];
  }
}

// ---------------------------------------------------------------------------
// Row softmax of the logits [BH, L, L] (float32) into weights of the
// activation dtype; with `causal`, query i sees keys 0..i.  One wavefront per
// row; the operation order is mtf.softmax's: exp(x - (log(sum(exp(x - max))) +
// max)).  A key that is not visible carries logit + (-1e9), whose exp is
// exactly 0 in float32, so it is left out of max and sum.
// ---------------------------------------------------------------------------
// With seq [B, L] (rows are (batch, head, query), H heads) a key is visible
// only if it carries the query's sequence id (transformer_layers.py:303-316).
// With rel_values [H, NB] and rel_bucket [2 L - 1] the logit of (query i, key j)
// gets the relative attention bias rel_values[head][rel_bucket[j - i + L - 1]]
// (transformer_layers.py:317-352) before the softmax.
template <typename T>
__global__ __launch_bounds__(256) void attention_softmax_kernel(
    const float* __restrict__ logits, T* __restrict__ weights, int64_t rows,
    int L, int causal, const int32_t* __restrict__ seq, int H,
    const T* __restrict__ rel_values, const int32_t* __restrict__ rel_bucket,
    int NB) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int i = (int)(row % L);
  const int visible = causal ? i + 1 : L;
  const int32_t* sb = seq ? seq + (row / L / H) * L : nullptr;
  const int my = sb ? sb[i] : 0;
  const float* xr = logits + row * L;
  const T* rv = rel_values ? rel_values + ((row / L) % H) * NB : nullptr;
  const int32_t* rb = rv ? rel_bucket + (L - 1 - i) : nullptr;   // rb[j]: bucket of j - i
  auto logit = [&](int j) {
    return rv ? xr[j] + load_f32<T>(rv + rb[j]) : xr[j];
  };
  float m = -INFINITY;
  for (int j = lane; j < visible; j += 64)
    if (!sb || sb[j] == my) m = fmaxf(m, logit(j));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  const float negm = -m;
  float sum = 0.f;
  for (int j = lane; j < visible; j += 64)
    if (!sb || sb[j] == my) sum += expf(logit(j) + negm);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const float neglse = -(logf(sum) + m);
  T* wr = weights + row * L;
  for (int j = lane; j < L; j += 64)
    store_f32<T>(wr + j, j < visible && (!sb || sb[j] == my)
                             ? expf(logit(j) + neglse) : 0.0f);
}

__global__ void fill_zero_f32_kernel(float* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

template <typename T>
__global__ void round_f32_kernel(const float* src, T* dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) store_f32<T>(dst + i, src[i]);
}

// Gradient of the relative attention bias values: dvalues[h][bucket] = sum over
// the batch and the (query, key) pairs of that bucket of dlogits (the gradient
// of mtf.gather, transformer_layers.py:351).  One wavefront per row of
// dlogits [B*H, L, L]; a block's four rows meet in an LDS histogram and go to
// the float32 accumulator acc [H, NB] with one atomic per bucket.
template <typename T>
__global__ __launch_bounds__(256) void relative_bias_backward_kernel(
    const T* __restrict__ dlogits, const int32_t* __restrict__ rel_bucket,
    float* __restrict__ acc, int64_t rows, int L, int H, int NB) {
  extern __shared__ float rb_hist[];           // [4][NB]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 4 * NB; i += 256) rb_hist[i] = 0.f;
  __syncthreads();
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row < rows) {
    const int i = (int)(row % L);
    const T* dr = dlogits + row * L;
    const int32_t* rb = rel_bucket + (L - 1 - i);
    for (int j = lane; j < L; j += 64) {
      const float v = load_f32<T>(dr + j);
      if (v != 0.f) atomicAdd(&rb_hist[wave * NB + rb[j]], v);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 4 * NB; i += 256) {
    const int w = i / NB, bkt = i - w * NB;
    const int64_t r = (int64_t)blockIdx.x * 4 + w;
    const float v = rb_hist[i];
    if (r < rows && v != 0.f)
      atomicAdd(acc + ((r / L) % H) * NB + bkt, v);
  }
}

// The same softmax for bf16 weights and rows of ITERS * 512 logits: a lane
// keeps its 8 * ITERS logits in registers (one pass over memory), reads them
// 32 bytes at a time and writes 16 bytes of weights at a time.
template <int ITERS>
__global__ __launch_bounds__(256) void attention_softmax_rows_kernel(
    const float* __restrict__ logits, bf16_t* __restrict__ weights,
    int64_t rows, int causal) {
  constexpr int L = ITERS * 512;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int visible = causal ? (int)(row % L) + 1 : L;
  const float* xr = logits + row * L;
  float v[ITERS][8];
  float m = -INFINITY;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int base = (it * 64 + lane) * 8;
    if (base < visible) {
      const float4 a = *reinterpret_cast<const float4*>(xr + base);
      const float4 b = *reinterpret_cast<const float4*>(xr + base + 4);
      const float t[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[it][j] = base + j < visible ? t[j] : -INFINITY;
        m = fmaxf(m, v[it][j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[it][j] = -INFINITY;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  const float negm = -m;
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it)
#pragma unroll
    for (int j = 0; j < 8; ++j) sum += expf(v[it][j] + negm);   // exp(-inf) = 0
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const float neglse = -(logf(sum) + m);
  bf16_t* wr = weights + row * L;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int base = (it * 64 + lane) * 8;
    uint4 o;
    bf16_t* os = reinterpret_cast<bf16_t*>(&o);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      store_f32<bf16_t>(os + j, expf(v[it][j] + neglse));
    *reinterpret_cast<uint4*>(wr + base) = o;
  }
}

// Picks the register-resident kernel where the row length allows it.
template <typename T>
static void launch_attention_softmax(const float* logits, T* weights,
                                     int64_t rows, int L, int causal,
                                     const int32_t* seq, int H,
                                     const void* rel_values,
                                     const int32_t* rel_bucket, int NB,
                                     hipStream_t st) {
  const unsigned blocks = (unsigned)((rows + 3) / 4);
  if (seq != nullptr || rel_values != nullptr)
    return attention_softmax_kernel<T><<<blocks, 256, 0, st>>>(
        logits, weights, rows, L, causal, seq, H, (const T*)rel_values,
        rel_bucket, NB);
  if constexpr (sizeof(T) == 2) {
    const bool aligned =
        (((uintptr_t)logits | (uintptr_t)weights) % 32) == 0;
    if (aligned && L == 512)
      return attention_softmax_rows_kernel<1><<<blocks, 256, 0, st>>>(
          logits, weights, rows, causal);
    if (aligned && L == 1024)
      return attention_softmax_rows_kernel<2><<<blocks, 256, 0, st>>>(
          logits, weights, rows, causal);
    if (aligned && L == 2048)
      return attention_softmax_rows_kernel<4><<<blocks, 256, 0, st>>>(
          logits, weights, rows, causal);
    if (aligned && L == 4096)
      return attention_softmax_rows_kernel<8><<<blocks, 256, 0, st>>>(
          logits, weights, rows, causal);
  }
  attention_softmax_kernel<T><<<blocks, 256, 0, st>>>(
      logits, weights, rows, L, causal, nullptr, H, nullptr, rel_bucket, NB);
}

template <typename T>
static int run_attention(const T* q, const T* k, const T* v, T* out, int B,
                         int L, int H, int D, int causal, const int32_t* seq,
                         const void* rel_values, const int32_t* rel_bucket,
                         int NB, int dtype, void* workspace, hipStream_t st) {
  const int BH = B * H;
  const size_t hd = (size_t)BH * L * D, ll = (size_t)BH * L * L;
  auto up = [](uintptr_t p) { return (p + 255) & ~(uintptr_t)255; };
  T* qh = (T*)up((uintptr_t)workspace);
  T* kh = (T*)up((uintptr_t)(qh + hd));
  T* vt = (T*)up((uintptr_t)(kh + hd));
  T* oh = (T*)up((uintptr_t)(vt + hd));
  float* logits = (float*)up((uintptr_t)(oh + hd));
  T* weights = (T*)up((uintptr_t)(logits + ll));
  const int64_t n = (int64_t)hd;
  const unsigned eb = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256
                                                         : 65536);
  split_heads_kernel<T><<<eb, 256, 0, st>>>(q, qh, B, L, H, D);
  MOE_CHECK_LAUNCH("self_attention (split q)");
  split_heads_kernel<T><<<eb, 256, 0, st>>>(k, kh, B, L, H, D);
  MOE_CHECK_LAUNCH("self_attention (split k)");
  dim3 tg((unsigned)((L + 31) / 32), (unsigned)((D + 31) / 32), (unsigned)BH);
  transpose_heads_kernel<T><<<tg, 256, 0, st>>>(v, vt, B, L, H, D);
  MOE_CHECK_LAUNCH("self_attention (transpose v)");
  int rc = batched_gemm_nt(qh, kh, logits, BH, L, L, D, dtype, true, st);
  if (rc != 0) return rc;
  const int64_t rows = (int64_t)BH * L;
  launch_attention_softmax<T>(logits, weights, rows, L, causal, seq, H,
                              rel_values, rel_bucket, NB, st);
  MOE_CHECK_LAUNCH("self_attention (softmax)");
  rc = batched_gemm_nt(weights, vt, oh, BH, L, D, L, dtype, false, st);
  if (rc != 0) return rc;
  merge_heads_kernel<T><<<eb, 256, 0, st>>>(oh, out, B, L, H, D);
  MOE_CHECK_LAUNCH("self_attention (merge)");
  return 0;
}

// ---------------------------------------------------------------------------
// Backward of the RMS norm y = x * r * scale, r = rsqrt(mean(x^2) + eps):
// with g = dy * scale, dx = r * g - x * r^3 * mean(g * x).  One wavefront per
// row, float32 arithmetic, one rounding; r goes to rstd[row] for the scale's
// gradient dscale[j] = sum_rows dy * x * r.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_backward_kernel(
    const T* __restrict__ x, const T* __restrict__ scale,
    const T* __restrict__ dy, T* __restrict__ dx, float* __restrict__ rstd,
    int64_t rows, int M, float inv_m, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * M;
  const T* gr = dy + row * M;
  float sumsq = 0.f, dot = 0.f;
  for (int i = lane; i < M; i += 64) {
    const float v = load_f32<T>(xr + i);
    sumsq = fmaf(v, v, sumsq);
    dot = fmaf(load_f32<T>(gr + i) * load_f32<T>(scale + i), v, dot);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sumsq += __shfl_xor(sumsq, off);
    dot += __shfl_xor(dot, off);
  }
  const float r = 1.0f / sqrtf(sumsq * inv_m + eps);
  const float c = r * r * r * dot * inv_m;
  if (lane == 0) rstd[row] = r;
  T* outr = dx + row * M;
  for (int i = lane; i < M; i += 64) {
    const float v = load_f32<T>(xr + i);
    const float g = load_f32<T>(gr + i) * load_f32<T>(scale + i);
    store_f32<T>(outr + i, g * r - v * c);
  }
}

// partial[chunk, j] = sum over the chunk's rows of dy * x * rstd
// bf16 rows of ITERS * 512 elements, 16-byte aligned: a wavefront keeps its row
// (x and g = dy * scale as float32) in registers, reads x and dy once with
// 16-byte loads and also carries the scale gradient's partial sums
// sum_rows dy * x * r for its rows, so the second pass over x and dy of the
// generic path drops out.  Wavefront w of the grid takes rows w, w + W, ...;
// the four wavefronts of a block add their partial sums in LDS (in wavefront
// order) and write partial[block][M].
template <int ITERS>
__global__ __launch_bounds__(256, 2) void rms_norm_backward_rows_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ scale,
    const bf16_t* __restrict__ dy, bf16_t* __restrict__ dx,
    float* __restrict__ partial, int64_t rows, float inv_m, float eps) {
  constexpr int M = ITERS * 512;
  __shared__ float red[M];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t stride = (int64_t)gridDim.x * 4;
  // x, dy and scale stay packed (two bf16 per register) and are unpacked where
  // they are used: 32 + 32 + 32 + 64 registers at 4096 columns
  uint32_t sc[ITERS][4];
  float acc[ITERS][8];
  auto lo = [](uint32_t w) { return __uint_as_float(w << 16); };
  auto hi = [](uint32_t w) { return __uint_as_float(w & 0xffff0000u); };
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const uint4 sv = *reinterpret_cast<const uint4*>(scale + (it * 64 + lane) * 8);
    sc[it][0] = sv.x; sc[it][1] = sv.y; sc[it][2] = sv.z; sc[it][3] = sv.w;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[it][j] = 0.f;
  }
  for (int64_t row = (int64_t)blockIdx.x * 4 + wave; row < rows; row += stride) {
    const bf16_t* xr = x + row * M;
    const bf16_t* gr = dy + row * M;
    uint32_t xv[ITERS][4], gv[ITERS][4];
    float sumsq = 0.f, dot = 0.f;
    // (the empty asm statements make the packed registers opaque, so that the
    // compiler unpacks them at each use instead of keeping 192 floats alive)
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(sc[it][j]));
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const uint4 a = load_streaming(
          reinterpret_cast<const uint4*>(xr + (it * 64 + lane) * 8));
      const uint4 b = load_streaming(
          reinterpret_cast<const uint4*>(gr + (it * 64 + lane) * 8));
      xv[it][0] = a.x; xv[it][1] = a.y; xv[it][2] = a.z; xv[it][3] = a.w;
      gv[it][0] = b.x; gv[it][1] = b.y; gv[it][2] = b.z; gv[it][3] = b.w;
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v0 = lo(xv[it][j]), v1 = hi(xv[it][j]);
        sumsq = fmaf(v0, v0, sumsq);
        dot = fmaf(lo(gv[it][j]) * lo(sc[it][j]), v0, dot);
        sumsq = fmaf(v1, v1, sumsq);
        dot = fmaf(hi(gv[it][j]) * hi(sc[it][j]), v1, dot);
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      sumsq += __shfl_xor(sumsq, off);
      dot += __shfl_xor(dot, off);
    }
    const float r = 1.0f / sqrtf(sumsq * inv_m + eps);
    const float c = r * r * r * dot * inv_m;
    bf16_t* outr = dx + row * M;
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        asm volatile("" : "+v"(sc[it][j]), "+v"(xv[it][j]), "+v"(gv[it][j]));
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v0 = lo(xv[it][j]), v1 = hi(xv[it][j]);
        const float d0 = lo(gv[it][j]), d1 = hi(gv[it][j]);
        o[j] = f32x2_to_bf16x2(d0 * lo(sc[it][j]) * r - v0 * c,
                               d1 * hi(sc[it][j]) * r - v1 * c);
        acc[it][2 * j] = fmaf(d0 * v0, r, acc[it][2 * j]);
        acc[it][2 * j + 1] = fmaf(d1 * v1, r, acc[it][2 * j + 1]);
      }
      uint4 ov;
      ov.x = o[0]; ov.y = o[1]; ov.z = o[2]; ov.w = o[3];
      store_streaming(reinterpret_cast<uint4*>(outr + (it * 64 + lane) * 8), ov);
    }
  }
  for (int w = 0; w < 4; ++w) {
    if (wave == w) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int col = (it * 64 + lane) * 8 + j;
          red[col] = w == 0 ? acc[it][j] : red[col] + acc[it][j];
        }
    }
    __syncthreads();
  }
  float* pr = partial + (int64_t)blockIdx.x * M;
  for (int i = threadIdx.x; i < M; i += 256) pr[i] = red[i];
}

constexpr int RMS_ROWS_BLOCKS = 512;   // two per CU

static bool rms_rows_path(int64_t rows, int M, int dtype, const void* x,
                          const void* scale, const void* dy, const void* dx) {
  return dtype == MESH_MOE_BF16 && M % 512 == 0 && M >= 512 && M <= 4096 &&
         rows >= 1 &&
         (((uintptr_t)x | (uintptr_t)scale | (uintptr_t)dy | (uintptr_t)dx) % 16 ==
          0);
}

template <typename T>
__global__ __launch_bounds__(256) void rms_norm_dscale_partial_kernel(
    const T* __restrict__ x, const T* __restrict__ dy,
    const float* __restrict__ rstd, float* __restrict__ partial, int64_t rows,
    int M, int64_t rows_per_chunk) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= M) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < rows ? r0 + rows_per_chunk : rows;
  float acc = 0.f;
  for (int64_t r = r0; r < r1; ++r)
    acc = fmaf(load_f32<T>(dy + r * M + j) * load_f32<T>(x + r * M + j),
               rstd[r], acc);
  partial[(int64_t)blockIdx.y * M + j] = acc;
}

// dscale[j] = sum over the chunks of partial[c][j].  A block takes 64 columns;
// its 16 wavefronts take every 16th chunk each (independent loads, eight in
// flight) and meet in LDS.  (One thread per column walking all chunks one after
// the other took 0.13 ms for 512 x 4096 partial sums: 16 blocks, each load
// waited for.)
constexpr int DSCALE_FINAL_THREADS = 1024;
template <typename T>
__global__ __launch_bounds__(DSCALE_FINAL_THREADS) void rms_norm_dscale_final_kernel(
    const float* __restrict__ partial, T* __restrict__ dscale, int chunks,
    int M) {
  __shared__ float part[16][64];
  const int col = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int j = blockIdx.x * 64 + col;
  float acc = 0.f;
  if (j < M) {
    int c = grp;
    for (; c + 7 * 16 < chunks; c += 8 * 16) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partial[(int64_t)(c + 16 * u) * M + j];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; c < chunks; c += 16) acc += partial[(int64_t)c * M + j];
  }
  part[grp][col] = acc;
  __syncthreads();
  if (grp == 0 && j < M) {
    float total = 0.f;
#pragma unroll
    for (int g = 0; g < 16; ++g) total += part[g][col];
    store_f32<T>(dscale + j, total);
  }
}

static int rms_norm_dscale_chunks(int64_t rows) {
  const int64_t c = (rows + 255) / 256;
  return (int)(c < 1 ? 1 : (c > 256 ? 256 : c));
}

// ---------------------------------------------------------------------------
// Backward of a softmax over the last dim from its output:
// dlogits = w * (dw - sum_k dw * w).  One wavefront per row, float32
// arithmetic, one rounding.  Where w is 0 (keys that are not visible) so is
// the result.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void softmax_backward_kernel(
    const T* __restrict__ w, const T* __restrict__ dw, T* __restrict__ dlogits,
    int64_t rows, int L) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* wr = w + row * L;
  const T* dr = dw + row * L;
  float dot = 0.f;
  for (int j = lane; j < L; j += 64)
    dot = fmaf(load_f32<T>(dr + j), load_f32<T>(wr + j), dot);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
  T* outr = dlogits + row * L;
  for (int j = lane; j < L; j += 64)
    store_f32<T>(outr + j, load_f32<T>(wr + j) * (load_f32<T>(dr + j) - dot));
}

// The same for bf16 rows of ITERS * 512 elements, both rows held in registers
// and moved 16 bytes at a time.
template <int ITERS>
__global__ __launch_bounds__(256) void softmax_backward_rows_kernel(
    const bf16_t* __restrict__ w, const bf16_t* __restrict__ dw,
    bf16_t* __restrict__ dlogits, int64_t rows) {
  constexpr int L = ITERS * 512;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const bf16_t* wr = w + row * L;
  const bf16_t* dr = dw + row * L;
  float wv[ITERS][8], dv[ITERS][8];
  float dot = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int base = (it * 64 + lane) * 8;
    const uint4 a = *reinterpret_cast<const uint4*>(wr + base);
    const uint4 b = *reinterpret_cast<const uint4*>(dr + base);
    const bf16_t* as = reinterpret_cast<const bf16_t*>(&a);
    const bf16_t* bs = reinterpret_cast<const bf16_t*>(&b);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      wv[it][j] = load_f32<bf16_t>(as + j);
      dv[it][j] = load_f32<bf16_t>(bs + j);
      dot = fmaf(dv[it][j], wv[it][j], dot);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
  bf16_t* outr = dlogits + row * L;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int base = (it * 64 + lane) * 8;
    uint4 o;
    bf16_t* os = reinterpret_cast<bf16_t*>(&o);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      store_f32<bf16_t>(os + j, wv[it][j] * (dv[it][j] - dot));
    *reinterpret_cast<uint4*>(outr + base) = o;
  }
}

// The attention weights alone, heads to the front: weights [B*H, L, L].
template <typename T>
static int run_attention_weights(const T* q, const T* k, T* weights, int B,
                                 int L, int H, int D, int causal,
                                 const int32_t* seq, const void* rel_values,
                                 const int32_t* rel_bucket, int NB, int dtype,
                                 void* workspace, hipStream_t st) {
  const int BH = B * H;
  const size_t hd = (size_t)BH * L * D;
  auto up = [](uintptr_t p) { return (p + 255) & ~(uintptr_t)255; };
  T* qh = (T*)up((uintptr_t)workspace);
  T* kh = (T*)up((uintptr_t)(qh + hd));
  float* logits = (float*)up((uintptr_t)(kh + hd));
  const int64_t n = (int64_t)hd;
  const unsigned eb = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256
                                                         : 65536);
  split_heads_kernel<T><<<eb, 256, 0, st>>>(q, qh, B, L, H, D);
  MOE_CHECK_LAUNCH("attention_weights (split q)");
  split_heads_kernel<T><<<eb, 256, 0, st>>>(k, kh, B, L, H, D);
  MOE_CHECK_LAUNCH("attention_weights (split k)");
  int rc = batched_gemm_nt(qh, kh, logits, BH, L, L, D, dtype, true, st);
  if (rc != 0) return rc;
  const int64_t rows = (int64_t)BH * L;
  launch_attention_softmax<T>(logits, weights, rows, L, causal, seq, H,
                              rel_values, rel_bucket, NB, st);
  MOE_CHECK_LAUNCH("attention_weights (softmax)");
  return 0;
}

// Dropout with the noise broadcast over the middle of three index ranges
// (ops.py:5832-5872 with a noise_shape that leaves dimensions of x out):
// out[o, m, i] = x[o, m, i] * noise[o, i], noise = (uniform < keep) ? 1 / keep
// : 0, or `noise_in` as given.  One thread per (o, m) row piece of up to eight
// consecutive i; bf16 rows whose length is a multiple of eight move 16 bytes.
template <typename T>
__global__ __launch_bounds__(256) void broadcast_dropout_kernel(
    const T* __restrict__ x, const T* __restrict__ uniform,
    const T* __restrict__ noise_in, float keep, float inv_keep,
    T* __restrict__ out, T* __restrict__ noise_out, int64_t outer, int64_t mid,
    int64_t inner, bool vec8) {
  const int64_t step = vec8 ? 8 : 1;
  const int64_t per_row = inner / step;
  const int64_t total = outer * mid * per_row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total;
       w += stride) {
    const int64_t i0 = (w % per_row) * step;
    const int64_t om = w / per_row;
    const int64_t o = om / mid;
    const int64_t xi = om * inner + i0;
    const int64_t ni = o * inner + i0;
    const bool writes_noise = noise_out != nullptr && om % mid == 0;
    if (vec8) {
      const uint4 xv = *reinterpret_cast<const uint4*>(x + xi);
      const uint4 sv = *reinterpret_cast<const uint4*>(
          (noise_in ? noise_in : uniform) + ni);
      const bf16_t* xs = reinterpret_cast<const bf16_t*>(&xv);
      const bf16_t* ss = reinterpret_cast<const bf16_t*>(&sv);
      uint4 ov, nv;
      bf16_t* os = reinterpret_cast<bf16_t*>(&ov);
      bf16_t* ns = reinterpret_cast<bf16_t*>(&nv);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sj = load_f32<bf16_t>(ss + j);
        const float noise = noise_in ? sj : (sj < keep ? inv_keep : 0.f);
        store_f32<bf16_t>(ns + j, noise);
        store_f32<bf16_t>(os + j, load_f32<bf16_t>(xs + j) * noise);
      }
      *reinterpret_cast<uint4*>(out + xi) = ov;
      if (writes_noise) *reinterpret_cast<uint4*>(noise_out + ni) = nv;
    } else {
      const float sj = load_f32<T>((noise_in ? noise_in : uniform) + ni);
      const float noise = noise_in ? sj : (sj < keep ? inv_keep : 0.f);
      store_f32<T>(out + xi, load_f32<T>(x + xi) * noise);
      if (writes_noise) store_f32<T>(noise_out + ni, noise);
    }
  }
}

}  // namespace mesh_moe

using namespace mesh_moe;

extern "C" int mesh_moe_broadcast_dropout(const void* x, const void* uniform,
                                          const void* noise_in, float keep_prob,
                                          void* out, void* noise_out,
                                          int64_t outer, int64_t mid,
                                          int64_t inner, int dtype,
                                          void* stream) {
  MOE_REQUIRE(x && out, MESH_MOE_E_ARG, "broadcast_dropout: null pointer");
  MOE_REQUIRE((uniform != nullptr) != (noise_in != nullptr), MESH_MOE_E_ARG,
              "broadcast_dropout: exactly one of uniform and noise_in");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "broadcast_dropout: bad dtype %d", dtype);
  MOE_REQUIRE(outer >= 1 && mid >= 1 && inner >= 1, MESH_MOE_E_ARG,
              "broadcast_dropout: bad sizes %lld x %lld x %lld",
              (long long)outer, (long long)mid, (long long)inner);
  MOE_REQUIRE(noise_in || (keep_prob > 0.f && keep_prob <= 1.f), MESH_MOE_E_ARG,
              "broadcast_dropout: keep_prob %g outside (0, 1]", keep_prob);
  MOE_REQUIRE(outer <= (int64_t)1 << 40 && mid <= (int64_t)1 << 40 &&
                  inner <= (int64_t)1 << 40 &&
                  (double)outer * (double)mid * (double)inner < 9.0e18,
              MESH_MOE_E_UNSUPPORTED, "broadcast_dropout: too many elements");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32) {
    const int64_t total = outer * mid * inner;
    const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256
                                                         : 65536);
    broadcast_dropout_kernel<float><<<blocks, 256, 0, st>>>(
        (const float*)x, (const float*)uniform, (const float*)noise_in,
        keep_prob, 1.f / keep_prob, (float*)out, (float*)noise_out, outer, mid,
        inner, false);
  } else {
    const uintptr_t ptrs = (uintptr_t)x | (uintptr_t)uniform |
                           (uintptr_t)noise_in | (uintptr_t)out |
                           (uintptr_t)noise_out;
    const bool vec8 = inner % 8 == 0 && ptrs % 16 == 0;
    const int64_t total = outer * mid * (vec8 ? inner / 8 : inner);
    const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256
                                                         : 65536);
    // the threshold and 1 / keep_prob are scalars of the activation dtype
    const float keep = round_bf16_host(keep_prob);
    broadcast_dropout_kernel<bf16_t><<<blocks, 256, 0, st>>>(
        (const bf16_t*)x, (const bf16_t*)uniform, (const bf16_t*)noise_in, keep,
        round_bf16_host(1.f / keep), (bf16_t*)out, (bf16_t*)noise_out, outer,
        mid, inner, vec8);
  }
  MOE_CHECK_LAUNCH("broadcast_dropout");
  return 0;
}

extern "C" size_t mesh_moe_rms_norm_backward_workspace_bytes(int64_t rows,
                                                            int M) {
  if (rows < 1 || M < 1) return 0;
  const size_t parts =
      (size_t)rms_norm_dscale_chunks(rows) > (size_t)RMS_ROWS_BLOCKS
          ? (size_t)rms_norm_dscale_chunks(rows) : (size_t)RMS_ROWS_BLOCKS;
  return ((size_t)rows * 4 + 255) / 256 * 256 + parts * (size_t)M * 4;
}

extern "C" int mesh_moe_rms_norm_backward(const void* x, const void* scale,
                                          const void* dy, void* dx,
                                          void* dscale, int64_t rows, int M,
                                          double epsilon, int dtype,
                                          void* workspace,
                                          size_t workspace_bytes,
                                          void* stream) {
  MOE_REQUIRE(x && scale && dy && dx && dscale && workspace, MESH_MOE_E_ARG,
              "rms_norm_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "rms_norm_backward: bad dtype %d", dtype);
  MOE_REQUIRE(rows >= 1 && M >= 1, MESH_MOE_E_ARG,
              "rms_norm_backward: bad sizes rows=%lld M=%d", (long long)rows,
              M);
  const int64_t blocks = (rows + 3) / 4;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "rms_norm_backward: too many rows (%lld)", (long long)rows);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_rms_norm_backward_workspace_bytes(rows, M),
              MESH_MOE_E_ARG, "rms_norm_backward: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  float* rstd = (float*)workspace;
  float* partial =
      (float*)((char*)workspace + ((size_t)rows * 4 + 255) / 256 * 256);
  const int chunks = rms_norm_dscale_chunks(rows);
  const int64_t per_chunk = (rows + chunks - 1) / chunks;
  const dim3 pg((unsigned)((M + 255) / 256), (unsigned)chunks);
  const float inv_m = (float)(1.0 / (double)M);
  if (rms_rows_path(rows, M, dtype, x, scale, dy, dx)) {
    const int nb = (int)(blocks < RMS_ROWS_BLOCKS ? blocks : RMS_ROWS_BLOCKS);
    const bf16_t *x_ = (const bf16_t*)x, *s_ = (const bf16_t*)scale,
                 *g_ = (const bf16_t*)dy;
    const float e_ = round_bf16_host((float)epsilon);
    switch (M / 512) {
#define MOE_RMS_ROWS(IT)                                                       \
  case IT:                                                                     \
    rms_norm_backward_rows_kernel<IT><<<nb, 256, 0, st>>>(                     \
        x_, s_, g_, (bf16_t*)dx, partial, rows, inv_m, e_);                    \
    break;
      MOE_RMS_ROWS(1) MOE_RMS_ROWS(2) MOE_RMS_ROWS(3) MOE_RMS_ROWS(4)
      MOE_RMS_ROWS(5) MOE_RMS_ROWS(6) MOE_RMS_ROWS(7) MOE_RMS_ROWS(8)
#undef MOE_RMS_ROWS
    }
    MOE_CHECK_LAUNCH("rms_norm_backward (rows)");
    rms_norm_dscale_final_kernel<bf16_t><<<(unsigned)((M + 63) / 64),
                                           DSCALE_FINAL_THREADS, 0, st>>>(
        partial, (bf16_t*)dscale, nb, M);
    MOE_CHECK_LAUNCH("rms_norm_backward (dscale)");
    return 0;
  }
  if (dtype == MESH_MOE_F32) {
    rms_norm_backward_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(
        (const float*)x, (const float*)scale, (const float*)dy, (float*)dx,
        rstd, rows, M, inv_m, (float)epsilon);
    MOE_CHECK_LAUNCH("rms_norm_backward");
    rms_norm_dscale_partial_kernel<float><<<pg, 256, 0, st>>>(
        (const float*)x, (const float*)dy, rstd, partial, rows, M, per_chunk);
    MOE_CHECK_LAUNCH("rms_norm_backward (dscale partial)");
    rms_norm_dscale_final_kernel<float><<<(unsigned)((M + 63) / 64),
                                          DSCALE_FINAL_THREADS, 0, st>>>(
        partial, (float*)dscale, chunks, M);
  } else {
    rms_norm_backward_kernel<bf16_t><<<(unsigned)blocks, 256, 0, st>>>(
        (const bf16_t*)x, (const bf16_t*)scale, (const bf16_t*)dy, (bf16_t*)dx,
        rstd, rows, M, inv_m, round_bf16_host((float)epsilon));
    MOE_CHECK_LAUNCH("rms_norm_backward");
    rms_norm_dscale_partial_kernel<bf16_t><<<pg, 256, 0, st>>>(
        (const bf16_t*)x, (const bf16_t*)dy, rstd, partial, rows, M, per_chunk);
    MOE_CHECK_LAUNCH("rms_norm_backward (dscale partial)");
    rms_norm_dscale_final_kernel<bf16_t><<<(unsigned)((M + 63) / 64),
                                           DSCALE_FINAL_THREADS, 0, st>>>(
        partial, (bf16_t*)dscale, chunks, M);
  }
  MOE_CHECK_LAUNCH("rms_norm_backward (dscale)");
  return 0;
}

extern "C" int mesh_moe_softmax_backward(const void* weights,
                                         const void* dweights, void* dlogits,
                                         int64_t rows, int L, int dtype,
                                         void* stream) {
  MOE_REQUIRE(weights && dweights && dlogits, MESH_MOE_E_ARG,
              "softmax_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "softmax_backward: bad dtype %d", dtype);
  MOE_REQUIRE(rows >= 1 && L >= 1, MESH_MOE_E_ARG,
              "softmax_backward: bad sizes rows=%lld L=%d", (long long)rows, L);
  const int64_t blocks = (rows + 3) / 4;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "softmax_backward: too many rows (%lld)", (long long)rows);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32)
    softmax_backward_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(
        (const float*)weights, (const float*)dweights, (float*)dlogits, rows,
        L);
  else {
    const bf16_t* w = (const bf16_t*)weights;
    const bf16_t* dw = (const bf16_t*)dweights;
    bf16_t* dl = (bf16_t*)dlogits;
    const unsigned nb = (unsigned)blocks;
    const bool aligned =
        (((uintptr_t)w | (uintptr_t)dw | (uintptr_t)dl) % 16) == 0;
    if (aligned && L == 512)
      softmax_backward_rows_kernel<1><<<nb, 256, 0, st>>>(w, dw, dl, rows);
    else if (aligned && L == 1024)
      softmax_backward_rows_kernel<2><<<nb, 256, 0, st>>>(w, dw, dl, rows);
    else if (aligned && L == 2048)
      softmax_backward_rows_kernel<4><<<nb, 256, 0, st>>>(w, dw, dl, rows);
    else if (aligned && L == 4096)
      softmax_backward_rows_kernel<8><<<nb, 256, 0, st>>>(w, dw, dl, rows);
    else
      softmax_backward_kernel<bf16_t><<<nb, 256, 0, st>>>(w, dw, dl, rows, L);
  }
  MOE_CHECK_LAUNCH("softmax_backward");
  return 0;
}

extern "C" size_t mesh_moe_attention_weights_workspace_bytes(int B, int L,
                                                             int H, int D,
                                                             int dtype) {
  if (B < 1 || L < 1 || H < 1 || D < 1 || !valid_dtype(dtype)) return 0;
  const size_t b = dtype_size(dtype);
  const size_t hd = (size_t)B * H * L * D, ll = (size_t)B * H * L * L;
  return 2 * hd * b + ll * 4 + 4 * 256;
}

extern "C" int mesh_moe_attention_weights(const void* q, const void* k,
                                          void* weights, int B, int L, int H,
                                          int D, int causal,
                                          const int32_t* sequence_id,
                                          const void* rel_values,
                                          const int32_t* rel_bucket,
                                          int num_buckets, int dtype,
                                          void* workspace,
                                          size_t workspace_bytes,
                                          void* stream) {
  MOE_REQUIRE(q && k && weights && workspace, MESH_MOE_E_ARG,
              "attention_weights: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "attention_weights: bad dtype %d", dtype);
  MOE_REQUIRE(B >= 1 && L >= 1 && H >= 1 && D >= 1, MESH_MOE_E_ARG,
              "attention_weights: bad sizes B=%d L=%d H=%d D=%d", B, L, H, D);
  MOE_REQUIRE((int64_t)B * H <= 65535, MESH_MOE_E_UNSUPPORTED,
              "attention_weights: batch * heads = %lld > 65535",
              (long long)B * H);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_attention_weights_workspace_bytes(B, L, H, D, dtype),
              MESH_MOE_E_ARG, "attention_weights: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32)
    return run_attention_weights<float>((const float*)q, (const float*)k,
                                        (float*)weights, B, L, H, D,
                                        causal ? 1 : 0, sequence_id, rel_values,
                                        rel_bucket, num_buckets, dtype,
                                        workspace, st);
  return run_attention_weights<bf16_t>((const bf16_t*)q, (const bf16_t*)k,
                                       (bf16_t*)weights, B, L, H, D,
                                       causal ? 1 : 0, sequence_id, rel_values,
                                       rel_bucket, num_buckets, dtype,
                                       workspace, st);
}

extern "C" int mesh_moe_rms_norm(const void* x, const void* scale, void* y,
                                 int64_t rows, int M, double epsilon, int dtype,
                                 void* stream) {
  MOE_REQUIRE(x && scale && y, MESH_MOE_E_ARG, "rms_norm: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "rms_norm: bad dtype %d",
              dtype);
  MOE_REQUIRE(rows >= 1 && M >= 1, MESH_MOE_E_ARG,
              "rms_norm: bad sizes rows=%lld M=%d", (long long)rows, M);
  const int64_t blocks = (rows + 3) / 4;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "rms_norm: too many rows (%lld)", (long long)rows);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MESH_MOE_F32) {
    rms_norm_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(
        (const float*)x, (const float*)scale, (float*)y, rows, M,
        (float)(1.0 / (double)M), (float)epsilon, false);
  } else {
    // Python scalars reach the reference's ops rounded to the tensor dtype
    const float inv_m = round_bf16_host((float)(1.0 / (double)M));
    const float eps = round_bf16_host((float)epsilon);
    const bool vec16 =
        M % 8 == 0 &&
        (((uintptr_t)x | (uintptr_t)scale | (uintptr_t)y) % 16 == 0);
    const bf16_t *xb = (const bf16_t*)x, *sb = (const bf16_t*)scale;
    bf16_t* yb = (bf16_t*)y;
    if (vec16 && M <= 1024)
      rms_norm_rows_kernel<2><<<(unsigned)blocks, 256, 0, st>>>(xb, sb, yb, rows,
                                                               M, inv_m, eps);
    else if (vec16 && M <= 2048)
      rms_norm_rows_kernel<4><<<(unsigned)blocks, 256, 0, st>>>(xb, sb, yb, rows,
                                                               M, inv_m, eps);
    else if (vec16 && M <= 4096)
      rms_norm_rows_kernel<8><<<(unsigned)blocks, 256, 0, st>>>(xb, sb, yb, rows,
                                                               M, inv_m, eps);
    else
      rms_norm_kernel<bf16_t><<<(unsigned)blocks, 256, 0, st>>>(xb, sb, yb, rows,
                                                                M, inv_m, eps,
                                                                vec16);
  }
  MOE_CHECK_LAUNCH("rms_norm");
  return 0;
}

extern "C" size_t mesh_moe_self_attention_workspace_bytes(int B, int L, int H,
                                                          int D, int dtype,
                                                          int relative_bias) {
  if (B < 1 || L < 1 || H < 1 || D < 1 || !valid_dtype(dtype)) return 0;
  if (flash_attention_supported(L, H, D, dtype, nullptr, nullptr, nullptr,
                                nullptr))
    return flash_attention_workspace_bytes(B, L, H, D, relative_bias != 0);
  const size_t b = dtype_size(dtype);
  const size_t hd = (size_t)B * H * L * D, ll = (size_t)B * H * L * L;
  return 4 * hd * b + ll * 4 + ll * b + 7 * 256;
}

extern "C" int mesh_moe_self_attention(const void* q, const void* k,
                                       const void* v, void* out, int B, int L,
                                       int H, int D, int causal,
                                       const int32_t* sequence_id,
                                       const void* rel_values,
                                       const int32_t* rel_bucket,
                                       int num_buckets, float* lse, int dtype,
                                       void* workspace, size_t workspace_bytes,
                                       void* stream) {
  MOE_REQUIRE(q && k && v && out && workspace, MESH_MOE_E_ARG,
              "self_attention: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "self_attention: bad dtype %d", dtype);
  MOE_REQUIRE(B >= 1 && L >= 1 && H >= 1 && D >= 1, MESH_MOE_E_ARG,
              "self_attention: bad sizes B=%d L=%d H=%d D=%d", B, L, H, D);
  MOE_REQUIRE((int64_t)B * H <= 65535, MESH_MOE_E_UNSUPPORTED,
              "self_attention: batch * heads = %lld > 65535",
              (long long)B * H);
  MOE_REQUIRE((rel_values == nullptr) == (rel_bucket == nullptr) &&
                  (rel_values == nullptr || num_buckets >= 1),
              MESH_MOE_E_ARG,
              "self_attention: rel_values, rel_bucket and num_buckets go "
              "together");
  MOE_REQUIRE(workspace_bytes >= mesh_moe_self_attention_workspace_bytes(
                                     B, L, H, D, dtype, rel_values != nullptr),
              MESH_MOE_E_ARG, "self_attention: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  if (flash_attention_supported(L, H, D, dtype, nullptr, nullptr, nullptr,
                                nullptr)) {
    // fused kernel: the logits stay on chip
    MOE_REQUIRE(flash_attention_supported(L, H, D, dtype, q, k, v, out),
                MESH_MOE_E_UNSUPPORTED,
                "self_attention: q, k, v, out must be 16-byte aligned");
    return flash_attention(q, k, v, out, B, L, H, D, causal ? 1 : 0,
                           sequence_id, rel_values, rel_bucket, num_buckets,
                           lse, workspace, st);
  }
  MOE_REQUIRE(lse == nullptr, MESH_MOE_E_UNSUPPORTED,
              "self_attention: lse is written by the fused kernel only (bf16, "
              "d_kv 64 or 128, L a multiple of 8)");
  if (dtype == MESH_MOE_F32)
    return run_attention<float>((const float*)q, (const float*)k,
                                (const float*)v, (float*)out, B, L, H, D,
                                causal ? 1 : 0, sequence_id, rel_values,
                                rel_bucket, num_buckets, dtype, workspace, st);
  return run_attention<bf16_t>((const bf16_t*)q, (const bf16_t*)k,
                               (const bf16_t*)v, (bf16_t*)out, B, L, H, D,
                               causal ? 1 : 0, sequence_id, rel_values,
                               rel_bucket, num_buckets, dtype, workspace, st);
}

// ---------------------------------------------------------------------------
// One decoding step of self-attention ("incremental" mode,
// transformer/transformer_layers.py:231-254, :289-296).  One block per
// (head, batch entry): the step's key and value rows go into the caches at
// row position[b]; logits q . k_m in float32 for m <= position[b], float32
// softmax in the reference's op order, weights rounded to the activation
// dtype, out = sum_m w_m v_m.  The caches are read once: HBM-bound.
//   q, k_new, v_new, out [B, H*D]; k_cache, v_cache [B, Lm, H*D] (updated in
//   place); position [B] int32 on the device.
// NT threads per block: four wavefronts, or sixteen when the grid has few
// blocks (each block must then keep more loads in flight to draw its share of
// the bandwidth).  Dynamic LDS: max(Lm, NT) + D + 16 + 8 NT floats.
// ---------------------------------------------------------------------------
template <typename T, int NT>
__global__ __launch_bounds__(NT) void attention_decode_kernel(
    const T* __restrict__ q, const T* __restrict__ k_new,
    const T* __restrict__ v_new, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int32_t* __restrict__ position,
    T* __restrict__ out, int Lm, int H, int D, int vec,
    const T* __restrict__ rel_values, const int32_t* __restrict__ rel_bucket,
    int NB) {
  extern __shared__ __attribute__((aligned(16))) float dec_smem[];
  float* wl = dec_smem;                     // [max(Lm, NT)] logits, then weights
  float* qs = wl + (Lm > NT ? Lm : NT);     // [D]
  float* red = qs + D;                      // [16]
  float* part = red + 16;                   // [8 NT] partial outputs (vec path)
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int64_t hd = (int64_t)H * D;
  const int pos = min(max(position[b], 0), Lm - 1);
  // relative attention bias of memory position j against the step's position
  // (transformer_layers.py:317-352): values[h][bucket[j - pos + Lm - 1]]
  const T* rel_h = rel_values ? rel_values + (int64_t)h * NB : nullptr;
  const int32_t* rel_b = rel_values ? rel_bucket + (Lm - 1 - pos) : nullptr;
  const T* qr = q + b * hd + (int64_t)h * D;
  const T* knr = k_new + b * hd + (int64_t)h * D;
  const T* vnr = v_new + b * hd + (int64_t)h * D;
  T* kc = k_cache + (int64_t)b * Lm * hd + (int64_t)h * D;
  T* vc = v_cache + (int64_t)b * Lm * hd + (int64_t)h * D;
  for (int d = tid; d < D; d += NT) {
    qs[d] = load_f32<T>(qr + d);
    kc[(int64_t)pos * hd + d] = knr[d];
    vc[(int64_t)pos * hd + d] = vnr[d];
  }
  __syncthreads();
  constexpr int VN = Vec16B<T>::N;
  // vec path: a row is CH 16-byte chunks, read by LPR lanes (a power of two
  // >= CH, <= 64); the block's G = NT / LPR lane groups take rows g, g + G, ..
  const int CH = D / VN;
  int LPR = 1;
  while (LPR < CH) LPR *= 2;
  const int G = NT / LPR, g = tid / LPR, c = tid % LPR;
  const bool lane_on = c < CH;
  // logits of the visible rows; row `pos` comes from the step's own key
  float m = -INFINITY;
  if (vec) {
    float qv[VN];
#pragma unroll
    for (int u = 0; u < VN; ++u) qv[u] = lane_on ? qs[c * VN + u] : 0.f;
    constexpr int UR = 4;                   // rows in flight per lane group
    for (int j0 = g; j0 <= pos; j0 += G * UR) {
      uint4 raw[UR];
#pragma unroll
      for (int r = 0; r < UR; ++r) {
        const int j = j0 + r * G;
        raw[r] = make_uint4(0, 0, 0, 0);
        if (lane_on && j <= pos) {
          const T* kr = j == pos ? knr : kc + (int64_t)j * hd;
          raw[r] = load_streaming(reinterpret_cast<const uint4*>(kr) + c);
        }
      }
#pragma unroll
      for (int r = 0; r < UR; ++r) {
        const int j = j0 + r * G;
        float f[VN];
        unpack16(raw[r], f, T());
        float acc = 0.f;
#pragma unroll
        for (int u = 0; u < VN; ++u) acc = fmaf(qv[u], f[u], acc);
        for (int off = LPR >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (j <= pos) {
          if (rel_h) acc += load_f32<T>(rel_h + rel_b[j]);
          if (c == 0) wl[j] = acc;
          m = fmaxf(m, acc);
        }
      }
    }
  } else {
    for (int j = tid; j <= pos; j += NT) {
      const T* kr = j == pos ? knr : kc + (int64_t)j * hd;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc = fmaf(qs[d], load_f32<T>(kr + d), acc);
      if (rel_h) acc += load_f32<T>(rel_h + rel_b[j]);
      wl[j] = acc;
      m = fmaxf(m, acc);
    }
  }
  auto block_all = [&](float v, bool is_max) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float o = __shfl_xor(v, off, 64);
      v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < NT / 64; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
  };
  m = block_all(m, true);
  const float negm = -m;
  float sum = 0.f;
  for (int j = tid; j <= pos; j += NT) sum += expf(wl[j] + negm);
  sum = block_all(sum, false);
  const float neglse = -(logf(sum) + m);
  for (int j = tid; j <= pos; j += NT)
    wl[j] = round_to<T>(expf(wl[j] + neglse));
  __syncthreads();
  T* orow = out + b * hd + (int64_t)h * D;
  if (vec) {
    // out = sum_j w_j v_j: every lane group sums its rows for its chunk, the
    // groups' partial sums meet in LDS
    float acc[VN];
#pragma unroll
    for (int u = 0; u < VN; ++u) acc[u] = 0.f;
    constexpr int UR = 4;
    for (int j0 = g; j0 <= pos; j0 += G * UR) {
      uint4 raw[UR];
      float w[UR];
#pragma unroll
      for (int r = 0; r < UR; ++r) {
        const int j = j0 + r * G;
        raw[r] = make_uint4(0, 0, 0, 0);
        w[r] = 0.f;
        if (lane_on && j <= pos) {
          const T* vr = j == pos ? vnr : vc + (int64_t)j * hd;
          raw[r] = load_streaming(reinterpret_cast<const uint4*>(vr) + c);
          w[r] = wl[j];
        }
      }
#pragma unroll
      for (int r = 0; r < UR; ++r) {
        float f[VN];
        unpack16(raw[r], f, T());
#pragma unroll
        for (int u = 0; u < VN; ++u) acc[u] = fmaf(w[r], f[u], acc[u]);
      }
    }
    if (lane_on) {
#pragma unroll
      for (int u = 0; u < VN; ++u) part[g * D + c * VN + u] = acc[u];
    }
    __syncthreads();
    for (int d = tid; d < D; d += NT) {
      float total = 0.f;
      for (int gg = 0; gg < G; ++gg) total += part[gg * D + d];
      store_f32<T>(orow + d, total);
    }
  } else {
    for (int d = tid; d < D; d += NT) {
      float acc = 0.f;
      for (int j = 0; j <= pos; ++j) {
        const T* vr = j == pos ? vnr : vc + (int64_t)j * hd;
        acc = fmaf(wl[j], load_f32<T>(vr + d), acc);
      }
      store_f32<T>(orow + d, acc);
    }
  }
}

extern "C" int mesh_moe_attention_decode(const void* q, const void* k_new,
                                         const void* v_new, void* k_cache,
                                         void* v_cache, const int32_t* position,
                                         void* out, int B, int Lm, int H, int D,
                                         const void* rel_values,
                                         const int32_t* rel_bucket,
                                         int num_buckets, int dtype,
                                         void* stream) {
  MOE_REQUIRE(q && k_new && v_new && k_cache && v_cache && position && out,
              MESH_MOE_E_ARG, "attention_decode: null pointer");
  MOE_REQUIRE((rel_values == nullptr) == (rel_bucket == nullptr) &&
                  (rel_values == nullptr || num_buckets >= 1),
              MESH_MOE_E_ARG,
              "attention_decode: rel_values, rel_bucket and num_buckets go "
              "together");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "attention_decode: bad dtype %d", dtype);
  MOE_REQUIRE(B >= 1 && Lm >= 1 && H >= 1 && D >= 1, MESH_MOE_E_ARG,
              "attention_decode: bad sizes B=%d Lm=%d H=%d D=%d", B, Lm, H, D);
  MOE_REQUIRE(B <= 65535, MESH_MOE_E_UNSUPPORTED,
              "attention_decode: batch %d > 65535", B);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)H, (unsigned)B);
  const size_t esz = dtype_size(dtype);
  // 16-byte row reads: whole chunks per row, at most 64 of them, aligned
  const int vec = ((size_t)D * esz) % 16 == 0 && (size_t)D * esz <= 1024 &&
                  (((uintptr_t)k_cache | (uintptr_t)k_new | (uintptr_t)v_cache |
                    (uintptr_t)v_new) % 16) == 0;
  // few blocks: four times the threads, i.e. the loads in flight, per block
  const bool wide = vec && (int64_t)H * B <= 512 && Lm >= 2048 &&
                    ((size_t)Lm + D + 16 + 8 * 1024) * sizeof(float) <= 150 * 1024;
  const int nt = wide ? 1024 : 256;
  const size_t floats =
      (size_t)(Lm > nt ? Lm : nt) + (size_t)D + 16 + 8 * (size_t)nt;
  const size_t smem = floats * sizeof(float);
  MOE_REQUIRE(smem <= 150 * 1024, MESH_MOE_E_UNSUPPORTED,
              "attention_decode: memory length %d does not fit in LDS", Lm);
#define MOE_DECODE(T, NT)                                                      \
  do {                                                                         \
    auto kern = attention_decode_kernel<T, NT>;                                \
    MOE_ALLOW_LDS(kern, smem);                                                 \
    kern<<<grid, NT, smem, st>>>((const T*)q, (const T*)k_new, (const T*)v_new, \
                                 (T*)k_cache, (T*)v_cache, position, (T*)out,  \
                                 Lm, H, D, vec, (const T*)rel_values,          \
                                 rel_bucket, num_buckets);                     \
  } while (0)
  if (dtype == MESH_MOE_F32) {
    if (wide) MOE_DECODE(float, 1024); else MOE_DECODE(float, 256);
  } else {
    if (wide) MOE_DECODE(bf16_t, 1024); else MOE_DECODE(bf16_t, 256);
  }
#undef MOE_DECODE
  MOE_CHECK_LAUNCH("attention_decode");
  return 0;
}

extern "C" int mesh_moe_relative_bias_backward(const void* dlogits,
                                               const int32_t* rel_bucket,
                                               void* dvalues, float* workspace,
                                               int B, int L, int H,
                                               int num_buckets, int dtype,
                                               void* stream) {
  MOE_REQUIRE(dlogits && rel_bucket && dvalues && workspace, MESH_MOE_E_ARG,
              "relative_bias_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "relative_bias_backward: bad dtype %d", dtype);
  MOE_REQUIRE(B >= 1 && L >= 1 && H >= 1 && num_buckets >= 1 &&
                  num_buckets <= 4096,
              MESH_MOE_E_ARG,
              "relative_bias_backward: bad sizes B=%d L=%d H=%d buckets=%d", B,
              L, H, num_buckets);
  const int64_t rows = (int64_t)B * H * L;
  const int64_t blocks = (rows + 3) / 4;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "relative_bias_backward: too many rows (%lld)", (long long)rows);
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = (int64_t)H * num_buckets;
  const unsigned fb = (unsigned)((n + 255) / 256);
  fill_zero_f32_kernel<<<fb, 256, 0, st>>>(workspace, n);
  MOE_CHECK_LAUNCH("relative_bias_backward (clear)");
  const size_t smem = sizeof(float) * 4 * (size_t)num_buckets;
  if (dtype == MESH_MOE_F32) {
    relative_bias_backward_kernel<float><<<(unsigned)blocks, 256, smem, st>>>(
        (const float*)dlogits, rel_bucket, workspace, rows, L, H, num_buckets);
    MOE_CHECK_LAUNCH("relative_bias_backward");
    round_f32_kernel<float><<<fb, 256, 0, st>>>(workspace, (float*)dvalues, n);
  } else {
    relative_bias_backward_kernel<bf16_t><<<(unsigned)blocks, 256, smem, st>>>(
        (const bf16_t*)dlogits, rel_bucket, workspace, rows, L, H, num_buckets);
    MOE_CHECK_LAUNCH("relative_bias_backward");
    round_f32_kernel<bf16_t><<<fb, 256, 0, st>>>(workspace, (bf16_t*)dvalues, n);
  }
  MOE_CHECK_LAUNCH("relative_bias_backward (round)");
  return 0;
}

extern "C" size_t mesh_moe_self_attention_backward_workspace_bytes(
    int B, int L, int H, int D, int dtype, int relative_bias) {
  if (B < 1 || L < 1 || H < 1 || D < 1 || !valid_dtype(dtype)) return 0;
  if (!flash_attention_supported(L, H, D, dtype, nullptr, nullptr, nullptr,
                                 nullptr))
    return 0;
  return flash_attention_backward_workspace_bytes(B, L, H, relative_bias != 0);
}

extern "C" int mesh_moe_self_attention_backward(
    const void* q, const void* k, const void* v, const void* dout, void* dq,
    void* dk, void* dv, int B, int L, int H, int D, int causal,
    const int32_t* sequence_id, const void* rel_values,
    const int32_t* rel_bucket, int num_buckets, void* dvalues, const void* out,
    const float* lse, int dtype, void* workspace, size_t workspace_bytes,
    void* stream) {
  MOE_REQUIRE(q && k && v && dout && dq && dk && dv && workspace, MESH_MOE_E_ARG,
              "self_attention_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "self_attention_backward: bad dtype %d", dtype);
  MOE_REQUIRE(B >= 1 && L >= 1 && H >= 1 && D >= 1, MESH_MOE_E_ARG,
              "self_attention_backward: bad sizes B=%d L=%d H=%d D=%d", B, L, H,
              D);
  MOE_REQUIRE((int64_t)B * H <= 65535, MESH_MOE_E_UNSUPPORTED,
              "self_attention_backward: batch * heads = %lld > 65535",
              (long long)B * H);
  MOE_REQUIRE((rel_values == nullptr) == (rel_bucket == nullptr) &&
                  (rel_values == nullptr) == (dvalues == nullptr) &&
                  (rel_values == nullptr || num_buckets >= 1),
              MESH_MOE_E_ARG,
              "self_attention_backward: rel_values, rel_bucket, num_buckets "
              "and dvalues go together");
  MOE_REQUIRE((out == nullptr) == (lse == nullptr) &&
                  ((uintptr_t)out % 16) == 0,
              MESH_MOE_E_ARG,
              "self_attention_backward: out (16-byte aligned) and lse go "
              "together");
  MOE_REQUIRE(flash_attention_supported(L, H, D, dtype, q, k, v, dout) &&
                  flash_attention_supported(L, H, D, dtype, dq, dk, dv, dout),
              MESH_MOE_E_UNSUPPORTED,
              "self_attention_backward: the fused kernels take bf16, d_kv 64 or "
              "128, L a multiple of 8 and 16-byte aligned tensors (L=%d D=%d)",
              L, D);
  MOE_REQUIRE(workspace_bytes >= flash_attention_backward_workspace_bytes(
                                     B, L, H, rel_values != nullptr),
              MESH_MOE_E_ARG, "self_attention_backward: workspace too small");
  return flash_attention_backward(q, k, v, dout, dq, dk, dv, B, L, H, D,
                                  causal ? 1 : 0, sequence_id, rel_values,
                                  rel_bucket, num_buckets, dvalues, out, lse,
                                  workspace, (hipStream_t)stream);
}
