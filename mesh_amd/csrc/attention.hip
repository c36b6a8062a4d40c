// Fused multi-head self-attention for gfx950 (bf16, d_kv 64 or 128).
//
// Same mathematics as the three-step form in block.hip (attention.attention,
// mesh_tensorflow/transformer/attention.py:27-88, float32 logits): logits =
// q . k in float32, keys after the query masked when causal, float32 softmax,
// weights rounded to bf16, outputs = weights . v with float32 accumulation.
// The logits never leave the chip: a block owns 128 queries of one (batch,
// head) and walks the keys 64 at a time, keeping the running row maximum, the
// running sum and the unnormalised outputs (rescaled when the maximum moves);
// the division by the sum comes last.  Against the reference's order
// (normalise, then round the weights) this rounds the unnormalised weights:
// the same 2^-9 relative error per weight, applied before instead of after a
// common factor.
//
// Matrix-core layout.  Both products are computed transposed so that a lane
// owns ONE query throughout:
//   S^T tile  = K tile (MFMA rows = keys)  x Q (MFMA columns = queries)
//   O^T tile  = V^T tile (rows = d)        x P (columns = queries)
// With v_mfma_f32_32x32x16_bf16, lane l then holds, for query l % 32, the
// logits of keys 8*(r/4) + 4*(l/32) + r%4 (r = accumulator register) -- the row
// maximum and sum are 16 in-lane operations plus one exchange with lane l^32,
// and the rescaling factor of a query is a per-lane scalar.  The bf16 weights
// go straight from the accumulator registers into the second product's
// operand registers: MFMA step u of O^T uses registers 8*(u%2) .. +7 of key
// sub-tile u/2, which makes its 16 k-indices the keys 16u + {0-3, 8-11} for
// the lower half-wave and 16u + {4-7, 12-15} for the upper one.  The V^T
// operand comes from the V tile as it lies in memory (rows = keys) through
// ds_read_b64_tr_b16: within 16 lanes, lane t addresses the 8 bytes at (key row
// t / 4, elements 4 (t % 4) ..) of a 4 x 16 block and lane i receives column i,
// i.e. four consecutive keys of one d -- two such reads are exactly the 4 + 4
// keys of a step, so no data moves between lanes and V is never transposed in
// memory.
//
// K and V tiles reach a two-stage LDS ring through global_load_lds_dwordx4; K
// rows with XOR-swizzled 16-byte chunks, V rows with their 64-byte units
// XOR-ed by the key index (bank conflicts of the transposing reads); the
// queries of a wavefront stay in registers.  The transposing reads are inline
// asm: the compiler puts a vmcnt(0) in front of the builtin form, which would
// drain the next tile's loads; lgkmcnt(0) stands before the MFMAs that use
// their results.
#include "common.h"
#include <type_traits>

namespace mesh_moe {

typedef __attribute__((ext_vector_type(8))) __bf16 fa_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float fa_f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t fa_u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t fa_u32x2_t;
typedef __attribute__((address_space(3))) void fa_lds_void_t;
typedef const __attribute__((address_space(1))) void fa_glb_void_t;

template <int D>
struct FlashCfg {
  static constexpr int BQ = 128, BK = 64, WAVES = 4, THREADS = 64 * WAVES;
  static constexpr int K_ROW = D * 2;              // bytes per key row
  static constexpr int K_BYTES = BK * K_ROW;
  static constexpr int V_ROW = D * 2;              // bytes per key row of V
  static constexpr int V_BYTES = BK * V_ROW;
  static constexpr int V_RPI = 1024 / V_ROW;       // key rows per load instr
  static constexpr int VCH = V_ROW / 16;           // 16-byte chunks per row
  static constexpr int V_UNITS = V_ROW / 64;       // 64-byte units per row
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE;
  static constexpr int KCH = K_ROW / 16;           // 16-byte chunks per key row
  static constexpr int K_RPI = 1024 / K_ROW;       // key rows per load instr
  static constexpr int K_INSTR = K_BYTES / 1024 / WAVES;
  static constexpr int V_INSTR = V_BYTES / 1024 / WAVES;
  static constexpr int DS = D / 16;                // MFMA steps over d_kv
  static constexpr int DT = D / 32;                // 32-row tiles of O^T
  static_assert(D == 64 || D == 128, "d_kv 64 or 128");
};

// chunk swizzles: slot p of a row holds chunk p ^ swz(row)
template <int KCH>
__device__ __forceinline__ int fa_kswz(int row) {
  return KCH == 16 ? (row & 15) : ((row & 7) ^ ((row >> 3) & 1));
}
// 64-byte unit p of key row `row` of the V tile holds unit p ^ fa_vswz(row):
// the four rows a transposing read touches land on different banks
template <int UNITS>
__device__ __forceinline__ int fa_vswz(int row) {
  return UNITS == 4 ? (row & 3) : ((row >> 1) & 1);
}

typedef short fa_i16x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16 at LDS byte address `addr` + OFF
template <int OFF>
__device__ __forceinline__ fa_i16x4_t fa_lds_read_tr16(uint32_t addr) {
  fa_i16x4_t v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// 2^x as one v_exp_f32 (results below the normal range flush to 0, which is
// what a softmax weight that small is anyway; exp2f() spends four more
// instructions on that range)
__device__ __forceinline__ float fa_exp2(float x) {
  return __builtin_amdgcn_exp2f(x);
}

// Which (tile, batch * head) a block works on.  Workgroups go to the 8 XCDs
// round-robin in launch order (x fastest), so with the plain mapping the tiles
// of one (batch, head) land on all of them and every XCD's L2 fetches that
// head's K and V for itself.  Here XCD x takes the heads x, x + 8, ... and runs
// all tiles of a head back to back: a head's K and V enter one L2 once.
__device__ __forceinline__ void fa_block_to_work(int n_tiles, int& tile, int& bh) {
  const int nbh = (int)gridDim.y;
  if (nbh % 8 == 0) {
    const int id = (int)blockIdx.x + n_tiles * (int)blockIdx.y;
    const int slot = id >> 3;
    bh = (slot / n_tiles) * 8 + (id & 7);
    tile = slot % n_tiles;
  } else {
    tile = (int)blockIdx.x;
    bh = (int)blockIdx.y;
  }
}

// STATS: instead of the outputs, write what the backward kernels need per
// query: lse = log of the softmax denominator (row maximum included) and
// delta = sum_d dout[q, d] * out[q, d] (= sum_k dweights * weights), both
// float32 [B*H, L].
// SEQ: a query sees only the keys that carry its sequence id (seq [B, L];
// transformer_layers.py:303-316): the ids of a key tile travel through LDS
// with the tile, a lane keeps its query's id in a register.
// BIAS: the relative attention bias (transformer_layers.py:317-352) is added to
// the float32 logits: tab [H, 2L-1] holds, per head, the bias of every distance
// key - query + L - 1.  A tile's logits need a window of BK + BQ - 1 entries of
// it, which travels through LDS with the tile.
template <int D, bool CAUSAL, bool STATS = false, bool SEQ = false,
          bool BIAS = false>
__global__ __launch_bounds__(256, 2) void flash_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, bf16_t* __restrict__ out, int L, int H,
    const bf16_t* __restrict__ dout, float* __restrict__ lse,
    float* __restrict__ delta, const int32_t* __restrict__ seq,
    const float* __restrict__ tab) {
  using Cfg = FlashCfg<D>;
  extern __shared__ __attribute__((aligned(16))) unsigned char fa_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int nq = (L + Cfg::BQ - 1) / Cfg::BQ;
  int tile_x, bh;
  fa_block_to_work(nq, tile_x, bh);
  const int qt = nq - 1 - tile_x;            // long (late) query tiles first
  const int b = bh / H, h = bh % H;
  const int q0 = qt * Cfg::BQ;
  const int64_t row_stride = (int64_t)H * D;               // elements
  const bf16_t* qb = q + ((int64_t)b * L) * row_stride + (int64_t)h * D;
  const bf16_t* kb = k + ((int64_t)b * L) * row_stride + (int64_t)h * D;
  const bf16_t* vb = v + ((int64_t)b * L) * row_stride + (int64_t)h * D;
  bf16_t* ob = out + ((int64_t)b * L) * row_stride + (int64_t)h * D;

  const int n_ktiles_all = (L + Cfg::BK - 1) / Cfg::BK;
  const int n_ktiles =
      CAUSAL ? min(n_ktiles_all, (q0 + Cfg::BQ - 1) / Cfg::BK + 1)
             : n_ktiles_all;

  // this lane's query (second MFMA operand of S^T): 8 consecutive d per step
  const int my_q = q0 + wave * 32 + l32;
  const int32_t* seq_b = SEQ ? seq + (int64_t)b * L : nullptr;
  int my_sid = 0, own_first = 0;
  bool own_uniform = true;
  if constexpr (SEQ) {
    my_sid = seq_b[min(my_q, L - 1)];
    own_first = __builtin_amdgcn_readfirstlane(my_sid);
    own_uniform = __ballot(my_sid != own_first) == 0ull;
  }
  // key ids of the two tile stages, behind the K / V ring; then the two
  // stages' windows of the bias table (192 floats each)
  int32_t* sid_s = reinterpret_cast<int32_t*>(fa_smem + Cfg::LDS_BYTES);
  const float* bias_s = reinterpret_cast<const float*>(fa_smem + Cfg::LDS_BYTES + 512);
  const float* tab_h = BIAS ? tab + (int64_t)h * (2 * L - 1) : nullptr;
  fa_bf16x8_t qf[Cfg::DS];
  {
    const bf16_t* qr = qb + (int64_t)min(my_q, L - 1) * row_stride + half * 8;
#pragma unroll
    for (int s = 0; s < Cfg::DS; ++s)
      qf[s] = *reinterpret_cast<const fa_bf16x8_t*>(qr + s * 16);
  }

  // direct-to-LDS loads of one K tile and one V tile
  auto load_tile = [&](int kt, int buf) {
    const int key0 = kt * Cfg::BK;
    unsigned char* base = fa_smem + buf * Cfg::STAGE;
#pragma unroll
    for (int j = 0; j < Cfg::K_INSTR; ++j) {
      const int g = wave * Cfg::K_INSTR + j;
      const int row = g * Cfg::K_RPI + lane / Cfg::KCH;
      const int c = (lane % Cfg::KCH) ^ fa_kswz<Cfg::KCH>(row);
      const bf16_t* src =
          kb + (int64_t)min(key0 + row, L - 1) * row_stride + c * 8;
      __builtin_amdgcn_global_load_lds((fa_glb_void_t*)src,
                                       (fa_lds_void_t*)(base + g * 1024), 16, 0,
                                       0);
    }
#pragma unroll
    for (int j = 0; j < Cfg::V_INSTR; ++j) {
      const int g = wave * Cfg::V_INSTR + j;
      const int row = g * Cfg::V_RPI + lane / Cfg::VCH;     // key
      const int p = lane % Cfg::VCH;
      const int c = (((p >> 2) ^ fa_vswz<Cfg::V_UNITS>(row)) << 2) | (p & 3);
      const bf16_t* src =
          vb + (int64_t)min(key0 + row, L - 1) * row_stride + c * 8;
      __builtin_amdgcn_global_load_lds(
          (fa_glb_void_t*)src,
          (fa_lds_void_t*)(base + Cfg::K_BYTES + g * 1024), 16, 0, 0);
    }
    if constexpr (SEQ) {
      if (wave == 0)
        __builtin_amdgcn_global_load_lds(
            (fa_glb_void_t*)(seq_b + min(key0 + lane, L - 1)),
            (fa_lds_void_t*)(fa_smem + Cfg::LDS_BYTES + buf * 256), 4, 0, 0);
    }
    if constexpr (BIAS) {
      // entry i of the window: distance key0 - (q0 + BQ - 1) + i (+ L - 1)
      if (wave >= 1) {
        const int i = (wave - 1) * 64 + lane;
        const int d = key0 - (q0 + Cfg::BQ - 1) + (L - 1) + i;
        __builtin_amdgcn_global_load_lds(
            (fa_glb_void_t*)(tab_h + min(max(d, 0), 2 * L - 2)),
            (fa_lds_void_t*)(fa_smem + Cfg::LDS_BYTES + 512 + buf * 768 +
                             (wave - 1) * 256),
            4, 0, 0);
      }
    }
  };

  fa_f32x16_t acc_o[Cfg::DT];
#pragma unroll
  for (int dt = 0; dt < Cfg::DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[dt][r] = 0.f;
  constexpr float NEG = -1e30f;
  constexpr float LOG2E = 1.4426950408889634f;
  float m_run = NEG;      // running maximum of this lane's query
  float l_part = 0.f;     // sum over this half-wave's keys

  load_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));   // vmcnt(0)
  __syncthreads();

  const int qw_first = q0 + wave * 32;
  for (int kt = 0; kt < n_ktiles; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < n_ktiles) load_tile(kt + 1, buf ^ 1);
    const int key0 = kt * Cfg::BK;
    // (a wavefront whose queries all precede this tile still runs it: every
    // weight comes out 0, which measured faster than skipping)
    // mask: diagonal and last tiles only, behind a branch the tiles in between
    // do not take
    bool need_mask =
        (CAUSAL && key0 + Cfg::BK - 1 > qw_first) || key0 + Cfg::BK > L;
    const int32_t* sid_t = sid_s + buf * 64;
    if constexpr (SEQ) {
      // (wave-uniform: any key of the tile or query of the wavefront with an
      // id other than the first query's)
      need_mask = need_mask || !own_uniform ||
                  __ballot(sid_t[lane] != own_first) != 0ull;
    }
    {
      const unsigned char* ks = fa_smem + buf * Cfg::STAGE;
      // S^T: two sub-tiles of 32 keys
      fa_f32x16_t acc_s[2];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_s[sub][r] = 0.f;
        const int row = sub * 32 + l32;
        const unsigned char* kr = ks + row * Cfg::K_ROW;
        const int sw = fa_kswz<Cfg::KCH>(row);
#pragma unroll
        for (int s = 0; s < Cfg::DS; ++s) {
          const fa_bf16x8_t kf = *reinterpret_cast<const fa_bf16x8_t*>(
              kr + (((2 * s + half) ^ sw) * 16));
          acc_s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              kf, qf[s], acc_s[sub], 0, 0, 0);
        }
      }
      if constexpr (BIAS) {
        // key key0 + kl + c against query q0 + 32 wave + l32
        const float* bw = bias_s + buf * 192 + (Cfg::BQ - 1 - wave * 32 - l32);
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
            for (int c = 0; c < 4; ++c)
              acc_s[sub][4 * r4 + c] += bw[sub * 32 + 8 * r4 + 4 * half + c];
      }
      // mask and row maximum
      if (need_mask) {
        // (the empty asm keeps the compiler from turning the branch into 64
        // selects that every tile would execute)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int kl = sub * 32 + 8 * r4 + 4 * half;     // key within tile
            int kid[4] = {0, 0, 0, 0};
            if constexpr (SEQ) {
              const int4 i4 = *reinterpret_cast<const int4*>(sid_t + kl);
              kid[0] = i4.x; kid[1] = i4.y; kid[2] = i4.z; kid[3] = i4.w;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              const int key = key0 + kl + c;
              const bool ok = key < L && (!CAUSAL || key <= my_q) &&
                              (!SEQ || kid[c] == my_sid);
              if (!ok) acc_s[sub][4 * r4 + c] = NEG;
            }
          }
        }
      }
      float mx = NEG;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc_s[sub][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = fa_exp2((m_run - m_new) * LOG2E);
      // (a tile with no visible key before any visible key was met: the
      // maximum is still the sentinel, and sentinel * log2e - sentinel * log2e
      // would leave the product's rounding error, ~1e22, as the exponent)
      const float mneg = m_new > 0.5f * NEG ? -m_new * LOG2E : -INFINITY;
      m_run = m_new;
      float psum = 0.f;
      fa_bf16x8_t pf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        uint32_t w[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int r = 8 * (u & 1) + 2 * c;
          const float p0 = fa_exp2(fmaf(acc_s[u >> 1][r], LOG2E, mneg));
          const float p1 = fa_exp2(fmaf(acc_s[u >> 1][r + 1], LOG2E, mneg));
          psum += p0 + p1;
          w[c] = f32x2_to_bf16x2(p0, p1);
        }
        fa_u32x4_t packed = {w[0], w[1], w[2], w[3]};
        pf[u] = __builtin_bit_cast(fa_bf16x8_t, packed);
      }
      l_part = l_part * alpha + psum;
      // the outputs are rescaled only when some query's maximum moved in this
      // tile (after the first few tiles it rarely does): alpha is exactly 1
      // otherwise and the 16 * D / 32 multiplications per lane drop out
      if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
        for (int dt = 0; dt < Cfg::DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc_o[dt][r] *= alpha;
      }
      // O^T += V^T . P: the V^T operand of step u, block dt is two
      // transposing reads of 4 key rows x 16 d each (per 16 lanes)
      {
        const uint32_t lds0 = (uint32_t)(size_t)(fa_lds_void_t*)fa_smem;
        const int t16 = lane & 15, g16 = lane >> 4;
        const int krow = 4 * (g16 >> 1) + (t16 >> 2);        // + 16 u (+ 8)
        const int dcol = (g16 & 1) * 16 + 4 * (t16 & 3);      // + 32 dt
        // row krow + 16 u + 8 j has the same fa_vswz as krow (multiples of 4
        // or 8 are added), so the unit swizzle is a per-lane constant
        const int sw = fa_vswz<Cfg::V_UNITS>(krow);
        uint32_t vaddr[Cfg::DT];
#pragma unroll
        for (int dt = 0; dt < Cfg::DT; ++dt) {
          const int col = dt * 32 + dcol;                     // element index
          vaddr[dt] = lds0 + buf * Cfg::STAGE + Cfg::K_BYTES +
                      krow * Cfg::V_ROW + (((col >> 5) ^ sw) << 6) +
                      (col & 31) * 2;
        }
        fa_i16x4_t vlo[2][4], vhi[2][4];
        auto read_v = [&](int dt, int slot) {
          const uint32_t a = vaddr[dt];
          vlo[slot][0] = fa_lds_read_tr16<0 * Cfg::V_ROW>(a);
          vhi[slot][0] = fa_lds_read_tr16<8 * Cfg::V_ROW>(a);
          vlo[slot][1] = fa_lds_read_tr16<16 * Cfg::V_ROW>(a);
          vhi[slot][1] = fa_lds_read_tr16<24 * Cfg::V_ROW>(a);
          vlo[slot][2] = fa_lds_read_tr16<32 * Cfg::V_ROW>(a);
          vhi[slot][2] = fa_lds_read_tr16<40 * Cfg::V_ROW>(a);
          vlo[slot][3] = fa_lds_read_tr16<48 * Cfg::V_ROW>(a);
          vhi[slot][3] = fa_lds_read_tr16<56 * Cfg::V_ROW>(a);
        };
        read_v(0, 0);
#pragma unroll
        for (int dt = 0; dt < Cfg::DT; ++dt) {
          const int cur = dt & 1;
          __builtin_amdgcn_sched_barrier(0);
          __builtin_amdgcn_s_waitcnt(0xc07f);      // lgkmcnt(0): block dt is here
          __builtin_amdgcn_sched_barrier(0);
          if (dt + 1 < Cfg::DT) read_v(dt + 1, cur ^ 1);
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const fa_bf16x8_t vf = __builtin_bit_cast(
                fa_bf16x8_t, __builtin_shufflevector(vlo[cur][u], vhi[cur][u], 0,
                                                     1, 2, 3, 4, 5, 6, 7));
            acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                vf, pf[u], acc_o[dt], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    // tile kt+1 has landed and everybody is done with tile kt
    __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));   // vmcnt(0)
    __syncthreads();
  }

  const float l_all = l_part + __shfl_xor(l_part, 32);
  const float inv = 1.0f / l_all;
  if constexpr (STATS) {
    const bf16_t* drow = dout + ((int64_t)b * L + min(my_q, L - 1)) * row_stride +
                         (int64_t)h * D;
    float dsum = 0.f;
#pragma unroll
    for (int dt = 0; dt < Cfg::DT; ++dt) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = dt * 32 + 8 * a + 4 * half;
        const uint2 g = *reinterpret_cast<const uint2*>(drow + d);
        dsum += acc_o[dt][4 * a + 0] * __uint_as_float(g.x << 16) +
                acc_o[dt][4 * a + 1] * __uint_as_float(g.x & 0xffff0000u) +
                acc_o[dt][4 * a + 2] * __uint_as_float(g.y << 16) +
                acc_o[dt][4 * a + 3] * __uint_as_float(g.y & 0xffff0000u);
      }
    }
    dsum += __shfl_xor(dsum, 32);
    if (my_q < L && half == 0) {
      lse[(int64_t)bh * L + my_q] = m_run + logf(l_all);
      delta[(int64_t)bh * L + my_q] = dsum * inv;
    }
    return;
  }
  if (my_q < L) {
    // (for a later backward pass that then needs no pass of its own for it)
    if (lse != nullptr && half == 0)
      lse[(int64_t)bh * L + my_q] = m_run + logf(l_all);
    bf16_t* orow = ob + (int64_t)my_q * row_stride;
#pragma unroll
    for (int dt = 0; dt < Cfg::DT; ++dt) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = dt * 32 + 8 * a + 4 * half;
        uint2 v;
        v.x = f32x2_to_bf16x2(acc_o[dt][4 * a + 0] * inv,
                              acc_o[dt][4 * a + 1] * inv);
        v.y = f32x2_to_bf16x2(acc_o[dt][4 * a + 2] * inv,
                              acc_o[dt][4 * a + 3] * inv);
        *reinterpret_cast<uint2*>(orow + d) = v;
      }
    }
  }
}

template <int D, bool CAUSAL, bool SEQ, bool BIAS>
static int launch_flash_one(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                            bf16_t* out, int B, int L, int H,
                            const int32_t* seq, const float* tab, float* lse,
                            hipStream_t st) {
  using Cfg = FlashCfg<D>;
  constexpr int LDS = Cfg::LDS_BYTES + 512 + 1536;  // + key ids, bias windows
  dim3 grid((unsigned)((L + Cfg::BQ - 1) / Cfg::BQ), (unsigned)(B * H));
  auto kern = flash_attention_kernel<D, CAUSAL, false, SEQ, BIAS>;
  MOE_ALLOW_LDS(kern, LDS);
  kern<<<grid, Cfg::THREADS, LDS, st>>>(q, k, v, out, L, H, nullptr, lse,
                                        nullptr, seq, tab);
  MOE_CHECK_LAUNCH("self_attention (fused)");
  return 0;
}

// Calls f(std::bool_constant<causal>, <seq>, <bias>) for run-time flags.
template <typename F>
static int flash_dispatch(bool causal, bool seq, bool bias, F&& f) {
  auto with_bias = [&](auto c, auto s) {
    return bias ? f(c, s, std::true_type()) : f(c, s, std::false_type());
  };
  auto with_seq = [&](auto c) {
    return seq ? with_bias(c, std::true_type()) : with_bias(c, std::false_type());
  };
  return causal ? with_seq(std::true_type()) : with_seq(std::false_type());
}

template <int D>
static int launch_flash(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                        bf16_t* out, int B, int L, int H, int causal,
                        const int32_t* seq, const float* tab, float* lse,
                        hipStream_t st) {
  return flash_dispatch(causal != 0, seq != nullptr, tab != nullptr,
                        [&](auto c, auto s, auto bi) {
    return launch_flash_one<D, decltype(c)::value, decltype(s)::value,
                            decltype(bi)::value>(q, k, v, out, B, L, H, seq, tab,
                                                 lse, st);
  });
}

// tab[h][d] = float(values[h][bucket[d]]) for the 2L-1 distances d = key -
// query + L - 1: the bias as mtf.gather of the activation-dtype values gives it
// (transformer_layers.py:343-350), widened to the logits' float32.
__global__ void relative_table_kernel(const bf16_t* __restrict__ values,
                                      const int32_t* __restrict__ bucket,
                                      float* __restrict__ tab, int n, int NB) {
  const int d = blockIdx.x * blockDim.x + threadIdx.x;
  if (d < n)
    tab[(int64_t)blockIdx.y * n + d] =
        load_f32<bf16_t>(values + (int64_t)blockIdx.y * NB + bucket[d]);
}

static int launch_relative_table(const void* values, const int32_t* bucket,
                                 float* tab, int L, int H, int NB,
                                 hipStream_t st) {
  const int n = 2 * L - 1;
  relative_table_kernel<<<dim3((unsigned)((n + 255) / 256), (unsigned)H), 256, 0,
                          st>>>((const bf16_t*)values, bucket, tab, n, NB);
  MOE_CHECK_LAUNCH("self_attention (bias table)");
  return 0;
}

static size_t relative_table_bytes(int L, int H) {
  return ((size_t)H * (2 * (size_t)L - 1) * sizeof(float) + 255) & ~(size_t)255;
}

bool flash_attention_supported(int L, int H, int D, int dtype, const void* q,
                               const void* k, const void* v, const void* out) {
  return dtype == MESH_MOE_BF16 && (D == 64 || D == 128) && L >= 8 &&
         L % 8 == 0 &&
         (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 ==
          0) && (int64_t)L * H * D < (1LL << 31);
}

size_t flash_attention_workspace_bytes(int B, int L, int H, int D,
                                       bool relative_bias) {
  (void)B; (void)D;
  // the bias table is the only scratch
  return 256 + (relative_bias ? relative_table_bytes(L, H) : 0);
}

int flash_attention(const void* q, const void* k, const void* v, void* out,
                    int B, int L, int H, int D, int causal,
                    const int32_t* sequence_id, const void* rel_values,
                    const int32_t* rel_bucket, int num_buckets, float* lse,
                    void* workspace, hipStream_t st) {
  float* tab = nullptr;
  if (rel_values != nullptr) {
    tab = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    const int rc = launch_relative_table(rel_values, rel_bucket, tab, L, H,
                                         num_buckets, st);
    if (rc != 0) return rc;
  }
  if (D == 128)
    return launch_flash<128>((const bf16_t*)q, (const bf16_t*)k,
                             (const bf16_t*)v, (bf16_t*)out, B, L, H, causal,
                             sequence_id, tab, lse, st);
  return launch_flash<64>((const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v,
                          (bf16_t*)out, B, L, H, causal, sequence_id, tab, lse,
                          st);
}

// ---------------------------------------------------------------------------
// Backward (the gradients of the two einsums and the softmax of
// attention.attention, mesh_tensorflow/transformer/attention.py:76-87, which
// mtf.gradients would assemble): with W = softmax(q . k) rounded to bf16,
//   dW = dout . v^T,  dS = W * (dW - delta)  rounded to bf16,
//   dv = W^T . dout,  dq = dS . k,  dk = dS^T . q.
// Nothing [L, L] reaches memory: W is recomputed per tile from q, k and the
// lse of the STATS pass, three times -- once per output, so that every output
// element is accumulated by one wavefront in a fixed order (no atomics, the
// same bits on every run):
//   BWD_DQ  a lane owns a query;  walks key tiles:    S, dW, dS, dq^T += K^T dS
//   BWD_DK  a lane owns a key;    walks query tiles:  S, dW, dS, dk^T += Q^T dS
//   BWD_DV  a lane owns a key;    walks query tiles:  S, W,      dv^T += dout^T W
// All three have the forward kernel's shape: "tile rows x own fragments" on
// the matrix cores with the own entity as MFMA column (so masks, lse and delta
// are per lane or per register), the bf16 result going from the accumulator
// registers straight into the operand registers of the second product, whose
// other operand is the streamed tile read through ds_read_b64_tr_b16.  A
// streamed tile that is read both ways (K in BWD_DQ, Q in BWD_DK) is loaded
// into LDS twice, once per swizzle.
// ---------------------------------------------------------------------------
enum { BWD_DQ = 0, BWD_DK = 1, BWD_DV = 2 };

template <int D>
struct FlashBwdCfg {
  static constexpr int BT = 64;                     // streamed rows per tile
  static constexpr int WAVES = 8, THREADS = 64 * WAVES, BOWN = 32 * WAVES;
  static constexpr int ROW = D * 2;                 // bytes per row
  static constexpr int TILE = BT * ROW;
  static constexpr int CH = ROW / 16, UNITS = ROW / 64, RPI = 1024 / ROW;
  static constexpr int INSTR = TILE / 1024 / WAVES; // loads per wave and tile copy
  static constexpr int DS = D / 16, DT = D / 32;
  // lse, delta, sequence ids of a tile, then its window of the bias table
  // (BT + BOWN - 1 distances, 320 floats)
  static constexpr int BIAS_AT = 3 * BT * 4;
  static constexpr int STATS_BYTES = BIAS_AT + 320 * 4;
  static constexpr int RING = 512;                  // floats, see dwin below
  static constexpr int stage_bytes(int what) {
    return (what == BWD_DV ? 2 : 3) * TILE + STATS_BYTES;
  }
  static_assert(BT + BOWN - 1 <= 320 && 320 + 3 * BT <= RING, "bias window");
  static_assert(D == 64 || D == 128, "d_kv 64 or 128");
  static_assert(INSTR >= 1, "a tile copy is at least one load per wavefront");
};

// BIAS: the logits are recomputed with the relative attention bias (tab as
// in the forward kernel); BWD_DQ also sums its dS along the diagonals into
// dtab [H, 2L-1] (float atomics), the gradient of tab.
template <int D, bool CAUSAL, int WHAT, bool SEQ, bool BIAS>
__global__ __launch_bounds__(512) void flash_attention_backward_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, const bf16_t* __restrict__ dout,
    const float* __restrict__ lse, const float* __restrict__ delta,
    bf16_t* __restrict__ grad, int L, int H, const int32_t* __restrict__ seq,
    const float* __restrict__ tab, float* __restrict__ dtab) {
  using Cfg = FlashBwdCfg<D>;
  constexpr bool OWN_Q = WHAT == BWD_DQ;
  constexpr int NCOPY = WHAT == BWD_DV ? 2 : 3;
  constexpr int STAGE = Cfg::stage_bytes(WHAT);
  constexpr float LOG2E = 1.4426950408889634f;
  extern __shared__ __attribute__((aligned(16))) unsigned char fb_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int n_own = (L + Cfg::BOWN - 1) / Cfg::BOWN;
  // long tiles first: late queries, early keys
  int tile_x, bh;
  fa_block_to_work(n_own, tile_x, bh);
  const int ot = OWN_Q && CAUSAL ? n_own - 1 - tile_x : tile_x;
  const int own0 = ot * Cfg::BOWN;
  const int b = bh / H, h = bh % H;
  const int64_t row_stride = (int64_t)H * D;
  const int64_t head_off = ((int64_t)b * L) * row_stride + (int64_t)h * D;
  // own rows supply the register fragments, streamed rows the LDS tiles
  const bf16_t* own1 = (OWN_Q ? q : k) + head_off;
  const bf16_t* own2 = (OWN_Q ? dout : v) + head_off;
  const bf16_t* str1 = (OWN_Q ? k : q) + head_off;
  const bf16_t* str2 = (OWN_Q ? v : dout) + head_off;
  const float* lse_b = lse + (int64_t)bh * L;
  const float* delta_b = delta + (int64_t)bh * L;
  const float* tab_h = BIAS ? tab + (int64_t)h * (2 * L - 1) : nullptr;

  const int nt_all = (L + Cfg::BT - 1) / Cfg::BT;
  int t_begin = 0, t_end = nt_all;
  if (CAUSAL) {
    if (OWN_Q) t_end = min(nt_all, (own0 + Cfg::BOWN - 1) / Cfg::BT + 1);
    else t_begin = own0 / Cfg::BT;
  }

  const int my = own0 + wave * 32 + l32;
  const int my_c = min(my, L - 1);
  fa_bf16x8_t f1[Cfg::DS], f2[WHAT == BWD_DV ? 1 : Cfg::DS];
  {
    const bf16_t* r1 = own1 + (int64_t)my_c * row_stride + half * 8;
    const bf16_t* r2 = own2 + (int64_t)my_c * row_stride + half * 8;
#pragma unroll
    for (int s = 0; s < Cfg::DS; ++s) {
      f1[s] = *reinterpret_cast<const fa_bf16x8_t*>(r1 + s * 16);
      if constexpr (WHAT != BWD_DV)
        f2[s] = *reinterpret_cast<const fa_bf16x8_t*>(r2 + s * 16);
    }
  }
  float my_lse2 = 0.f, my_delta = 0.f;
  if constexpr (OWN_Q) {
    my_lse2 = lse_b[my_c] * LOG2E;
    my_delta = delta_b[my_c];
  }
  const int32_t* seq_b = SEQ ? seq + (int64_t)b * L : nullptr;
  int my_sid = 0, own_first = 0;
  bool own_uniform = true;
  if constexpr (SEQ) {
    my_sid = seq_b[my_c];
    own_first = __builtin_amdgcn_readfirstlane(my_sid);
    own_uniform = __ballot(my_sid != own_first) == 0ull;
  }

  // one tile copy: rows of `src` from row0, chunk-swizzled for row reads
  // (TR = false) or unit-swizzled for transposing reads (TR = true)
  auto load_copy = [&](const bf16_t* src, int row0, unsigned char* dst,
                       auto tr_c) {
    constexpr bool TR = decltype(tr_c)::value;
#pragma unroll
    for (int j = 0; j < Cfg::INSTR; ++j) {
      const int g = wave * Cfg::INSTR + j;
      const int row = g * Cfg::RPI + lane / Cfg::CH;
      const int p = lane % Cfg::CH;
      const int c = TR ? ((((p >> 2) ^ fa_vswz<Cfg::UNITS>(row)) << 2) | (p & 3))
                       : (p ^ fa_kswz<Cfg::CH>(row));
      const bf16_t* a = src + (int64_t)min(row0 + row, L - 1) * row_stride + c * 8;
      __builtin_amdgcn_global_load_lds((fa_glb_void_t*)a,
                                       (fa_lds_void_t*)(dst + g * 1024), 16, 0, 0);
    }
  };
  auto load_tile = [&](int t, int buf) {
    const int row0 = t * Cfg::BT;
    unsigned char* base = fb_smem + buf * STAGE;
    load_copy(str1, row0, base, std::false_type());
    if constexpr (WHAT == BWD_DV) {
      load_copy(str2, row0, base + Cfg::TILE, std::true_type());
    } else {
      load_copy(str1, row0, base + Cfg::TILE, std::true_type());
      load_copy(str2, row0, base + 2 * Cfg::TILE, std::false_type());
    }
    if constexpr (!OWN_Q) {
      // lse and delta of the tile's queries: one 4-byte load per lane
      if (wave < 2) {
        const float* a = (wave == 0 ? lse_b : delta_b) + min(row0 + lane, L - 1);
        __builtin_amdgcn_global_load_lds(
            (fa_glb_void_t*)a,
            (fa_lds_void_t*)(base + NCOPY * Cfg::TILE + wave * 256), 4, 0, 0);
      }
    }
    if constexpr (SEQ) {
      if (wave == 2)
        __builtin_amdgcn_global_load_lds(
            (fa_glb_void_t*)(seq_b + min(row0 + lane, L - 1)),
            (fa_lds_void_t*)(base + NCOPY * Cfg::TILE + 512), 4, 0, 0);
    }
    if constexpr (BIAS) {
      // entry i of the window: the smallest distance key - query (+ L - 1)
      // between the tile and the block's own rows, plus i
      if (wave >= 3) {
        const int i = (wave - 3) * 64 + lane;
        const int d = (OWN_Q ? row0 - (own0 + Cfg::BOWN - 1)
                             : own0 - (row0 + Cfg::BT - 1)) + (L - 1) + i;
        __builtin_amdgcn_global_load_lds(
            (fa_glb_void_t*)(tab_h + min(max(d, 0), 2 * L - 2)),
            (fa_lds_void_t*)(base + NCOPY * Cfg::TILE + Cfg::BIAS_AT +
                             (wave - 3) * 256),
            4, 0, 0);
      }
    }
  };
  // BWD_DQ with BIAS: dS summed along the diagonals.  Within a wavefront the
  // 32 queries x 64 keys of a tile span the distances e = key - query in
  // [-31, 63].  Each value is rotated (ds_bpermute, inside its half-wave) to
  // lane m = (query - key) mod 32, which then only ever sees e = -m + 32 n,
  // n = 0, 1, 2: three accumulators per lane (ra0-2) take a tile's 32 values
  // per lane; at the end of the tile n = 0 and 1 are complete (the next tile
  // is 64 keys on: its n = 0 is this tile's n = 2) and go to dwin with ONE LDS
  // atomic per lane -- LDS float atomics are slow: one per value took seven
  // times the rest of the kernel.
  // dwin is a ring over the distances relative to the first tile's window
  // start: a tile adds into 320 consecutive entries, the window moves up by BT
  // per tile, and the BT entries it leaves behind are complete: one wavefront
  // moves them to dtab during the next tile (they are reused three tiles
  // later).
  float* dwin = reinterpret_cast<float*>(fb_smem + 2 * STAGE);
  float* dtab_h = nullptr;
  if constexpr (BIAS && OWN_Q) {
    dtab_h = dtab + (int64_t)h * (2 * L - 1);
    if (tid < Cfg::RING) dwin[tid] = 0.f;
  }
  auto flush_dwin = [&](int chunk) {   // 64 ring entries from distance chunk * BT
    const int slot = ((chunk * Cfg::BT) & (Cfg::RING - 1)) + lane;
    const float val = dwin[slot];
    dwin[slot] = 0.f;
    const int d = chunk * Cfg::BT - (own0 + Cfg::BOWN - 1) + (L - 1) + lane;
    if (val != 0.f && d >= 0 && d <= 2 * L - 2) atomicAdd(dtab_h + d, val);
  };
  float ra0 = 0.f, ra1 = 0.f, ra2 = 0.f;
  const int rot_m = l32 + 4 * half;        // lane m takes key column c from lane
  const int rot_hb = half << 7;            // (m + c) mod 32 of its half-wave

  fa_f32x16_t acc[Cfg::DT];
#pragma unroll
  for (int dt = 0; dt < Cfg::DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

  if (t_begin < t_end) load_tile(t_begin, 0);
  __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));   // vmcnt(0)
  __syncthreads();

  const int ow_first = own0 + wave * 32, ow_last = ow_first + 31;
  const uint32_t lds0 = (uint32_t)(size_t)(fa_lds_void_t*)fb_smem;
  const int t16 = lane & 15, g16 = lane >> 4;
  const int krow = 4 * (g16 >> 1) + (t16 >> 2);
  const int dcol = (g16 & 1) * 16 + 4 * (t16 & 3);
  const int tsw = fa_vswz<Cfg::UNITS>(krow);
  uint32_t toff[Cfg::DT];     // byte offset of this lane's transposing reads
#pragma unroll
  for (int dt = 0; dt < Cfg::DT; ++dt) {
    const int col = dt * 32 + dcol;
    toff[dt] = krow * Cfg::ROW + (((col >> 5) ^ tsw) << 6) + (col & 31) * 2;
  }

  for (int t = t_begin; t < t_end; ++t) {
    const int buf = (t - t_begin) & 1;
    if (t + 1 < t_end) load_tile(t + 1, buf ^ 1);
    const int row0 = t * Cfg::BT;
    const unsigned char* t1r = fb_smem + buf * STAGE;
    const unsigned char* t2r = t1r + 2 * Cfg::TILE;           // BWD_DQ, BWD_DK
    const uint32_t ttr = lds0 + buf * STAGE + Cfg::TILE;      // the copy read transposed
    const float* st = reinterpret_cast<const float*>(t1r + NCOPY * Cfg::TILE);
    bool need_mask =
        (CAUSAL && (OWN_Q ? row0 + Cfg::BT - 1 > ow_first : row0 < ow_last)) ||
        row0 + Cfg::BT > L;
    const int32_t* sid_t = reinterpret_cast<const int32_t*>(st + 2 * Cfg::BT);
    if constexpr (SEQ) {
      need_mask = need_mask || !own_uniform ||
                  __ballot(sid_t[lane] != own_first) != 0ull;
    }
    // this lane's view of the tile's bias window: entry of streamed row j is
    // bw[j] (own queries) or bw[-j] (own keys)
    const float* bw = nullptr;
    if constexpr (BIAS)
      bw = reinterpret_cast<const float*>(t1r + NCOPY * Cfg::TILE + Cfg::BIAS_AT) +
           (OWN_Q ? Cfg::BOWN - 1 - (wave * 32 + l32)
                  : wave * 32 + l32 + Cfg::BT - 1);
    if constexpr (BIAS && OWN_Q) {
      if (t > t_begin && wave == ((t - 1) & 7)) flush_dwin(t - 1);
    }

    auto do_sub = [&](auto sub_c) {
      constexpr int SUB = decltype(sub_c)::value;
      fa_f32x16_t acc_s, acc_dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc_s[r] = 0.f; acc_dp[r] = 0.f; }
      const int row = SUB * 32 + l32;
      const int sw = fa_kswz<Cfg::CH>(row);
      {
        const unsigned char* rr = t1r + row * Cfg::ROW;
#pragma unroll
        for (int s = 0; s < Cfg::DS; ++s) {
          const fa_bf16x8_t a = *reinterpret_cast<const fa_bf16x8_t*>(
              rr + (((2 * s + half) ^ sw) * 16));
          acc_s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, f1[s], acc_s, 0, 0, 0);
        }
      }
      if constexpr (WHAT != BWD_DV) {
        const unsigned char* rr = t2r + row * Cfg::ROW;
#pragma unroll
        for (int s = 0; s < Cfg::DS; ++s) {
          const fa_bf16x8_t a = *reinterpret_cast<const fa_bf16x8_t*>(
              rr + (((2 * s + half) ^ sw) * 16));
          acc_dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, f2[s], acc_dp, 0, 0, 0);
        }
      }
      if constexpr (BIAS) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int j = SUB * 32 + 8 * r4 + 4 * half + c;
            acc_s[4 * r4 + c] += OWN_Q ? bw[j] : bw[-j];
          }
      }
      // weights (and their gradient) of this lane's own entity against the
      // 16 streamed rows SUB * 32 + 8 (r / 4) + 4 half + r % 4
      float w[16];
      if constexpr (OWN_Q) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fa_exp2(fmaf(acc_s[r], LOG2E, -my_lse2));
          w[r] = p * (acc_dp[r] - my_delta);
        }
      } else {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int j = SUB * 32 + 8 * r4 + 4 * half;
          const float4 l4 = *reinterpret_cast<const float4*>(st + j);
          const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
          float dv4[4] = {0.f, 0.f, 0.f, 0.f};
          if constexpr (WHAT == BWD_DK) {
            const float4 d4 = *reinterpret_cast<const float4*>(st + Cfg::BT + j);
            dv4[0] = d4.x; dv4[1] = d4.y; dv4[2] = d4.z; dv4[3] = d4.w;
          }
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int r = 4 * r4 + c;
            const float p = fa_exp2(fmaf(acc_s[r], LOG2E, -lv[c] * LOG2E));
            w[r] = WHAT == BWD_DV ? p : p * (acc_dp[r] - dv4[c]);
          }
        }
      }
      if (need_mask) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int jl = SUB * 32 + 8 * r4 + 4 * half;       // row within tile
          int sid4[4] = {0, 0, 0, 0};
          if constexpr (SEQ) {
            const int4 i4 = *reinterpret_cast<const int4*>(sid_t + jl);
            sid4[0] = i4.x; sid4[1] = i4.y; sid4[2] = i4.z; sid4[3] = i4.w;
          }
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int sr = row0 + jl + c;
            const bool ok = sr < L &&
                            (!CAUSAL || (OWN_Q ? sr <= my : my <= sr)) &&
                            (!SEQ || sid4[c] == my_sid);
            if (!ok) w[4 * r4 + c] = 0.f;
          }
        }
      }
      if constexpr (BIAS && OWN_Q) {
        if (ow_last >= L) {          // rows past the end carry no gradient
          asm volatile("" ::: "memory");
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (my >= L) w[r] = 0.f;
        }
        // register r holds key SUB * 32 + c, c = 8 (r / 4) + r % 4 + 4 half: in
        // lane m it comes from query (m + c) mod 32, at distance
        // -m + 32 (SUB + [m + c >= 32])
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c0 = 8 * (r >> 2) + (r & 3);
          const int from = (((rot_m + c0) & 31) << 2) | rot_hb;
          const float val = __int_as_float(
              __builtin_amdgcn_ds_bpermute(from, __float_as_int(w[r])));
          const float up = rot_m >= 32 - c0 ? val : 0.f;
          hi += up;
          lo += val - up;
        }
        if constexpr (SUB == 0) { ra0 += lo; ra1 += hi; }
        else { ra1 += lo; ra2 += hi; }
      }
      fa_bf16x8_t wf[2];
#pragma unroll
      for (int uu = 0; uu < 2; ++uu) {
        uint32_t pk[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
          pk[c] = f32x2_to_bf16x2(w[8 * uu + 2 * c], w[8 * uu + 2 * c + 1]);
        fa_u32x4_t packed = {pk[0], pk[1], pk[2], pk[3]};
        wf[uu] = __builtin_bit_cast(fa_bf16x8_t, packed);
      }
      // acc^T += (streamed tile)^T . w over the 32 streamed rows of this SUB:
      // MFMA step uu covers rows SUB * 32 + 16 uu + {0-3, 8-11} (+ 4 for the
      // upper half-wave), two transposing reads each
      fa_i16x4_t lo[2][2], hi[2][2];
      auto read_t = [&](int dt, int slot) {
        const uint32_t a = ttr + toff[dt];
        lo[slot][0] = fa_lds_read_tr16<(SUB * 32 + 0) * Cfg::ROW>(a);
        hi[slot][0] = fa_lds_read_tr16<(SUB * 32 + 8) * Cfg::ROW>(a);
        lo[slot][1] = fa_lds_read_tr16<(SUB * 32 + 16) * Cfg::ROW>(a);
        hi[slot][1] = fa_lds_read_tr16<(SUB * 32 + 24) * Cfg::ROW>(a);
      };
      read_t(0, 0);
#pragma unroll
      for (int dt = 0; dt < Cfg::DT; ++dt) {
        const int cur = dt & 1;
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0)
        __builtin_amdgcn_sched_barrier(0);
        if (dt + 1 < Cfg::DT) read_t(dt + 1, cur ^ 1);
#pragma unroll
        for (int uu = 0; uu < 2; ++uu) {
          const fa_bf16x8_t tf = __builtin_bit_cast(
              fa_bf16x8_t, __builtin_shufflevector(lo[cur][uu], hi[cur][uu], 0, 1,
                                                   2, 3, 4, 5, 6, 7));
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tf, wf[uu], acc[dt], 0,
                                                            0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    do_sub(std::integral_constant<int, 0>());
    do_sub(std::integral_constant<int, 1>());
    if constexpr (BIAS && OWN_Q) {
      // the lower half-wave hands in n = 0 (e = -m), the upper one n = 1
      // (e = 32 - m), each the sum of both halves' accumulators
      const float got = __shfl_xor(half == 0 ? ra1 : ra0, 32);
      const float mine = (half == 0 ? ra0 : ra1) + got;
      const int rel = t * Cfg::BT + Cfg::BOWN - 1 - 32 * wave + 32 * half - l32;
      atomicAdd(dwin + (rel & (Cfg::RING - 1)), mine);
      ra0 = ra2;
      ra1 = 0.f;
      ra2 = 0.f;
    }

    __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));   // vmcnt(0): tile t+1 is here
    __syncthreads();
  }
  if constexpr (BIAS && OWN_Q) {
    // n = 2 of the last tile, then what its window still holds: five chunks
    if (t_end > t_begin) {
      const int rel = t_end * Cfg::BT + Cfg::BOWN - 1 - 32 * wave - l32;
      atomicAdd(dwin + (rel & (Cfg::RING - 1)), ra0);
      __syncthreads();
      if (wave < 5) flush_dwin(t_end - 1 + wave);
    }
  }

  if (my < L) {
    bf16_t* orow = grad + head_off + (int64_t)my * row_stride;
#pragma unroll
    for (int dt = 0; dt < Cfg::DT; ++dt) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int d = dt * 32 + 8 * a + 4 * half;
        uint2 o;
        o.x = f32x2_to_bf16x2(acc[dt][4 * a + 0], acc[dt][4 * a + 1]);
        o.y = f32x2_to_bf16x2(acc[dt][4 * a + 2], acc[dt][4 * a + 3]);
        *reinterpret_cast<uint2*>(orow + d) = o;
      }
    }
  }
}

template <int D, bool CAUSAL, int WHAT, bool SEQ, bool BIAS>
static int launch_flash_backward_one(const bf16_t* q, const bf16_t* k,
                                     const bf16_t* v, const bf16_t* dout,
                                     const float* lse, const float* delta,
                                     bf16_t* grad, int B, int L, int H,
                                     const int32_t* seq, const float* tab,
                                     float* dtab, hipStream_t st) {
  using Cfg = FlashBwdCfg<D>;
  constexpr int LDS = 2 * Cfg::stage_bytes(WHAT) +
                      (BIAS && WHAT == BWD_DQ ? Cfg::RING * 4 : 0);
  dim3 grid((unsigned)((L + Cfg::BOWN - 1) / Cfg::BOWN), (unsigned)(B * H));
  auto kern = flash_attention_backward_kernel<D, CAUSAL, WHAT, SEQ, BIAS>;
  MOE_ALLOW_LDS(kern, LDS);
  kern<<<grid, Cfg::THREADS, LDS, st>>>(q, k, v, dout, lse, delta, grad, L, H,
                                        seq, tab, dtab);
  MOE_CHECK_LAUNCH("self_attention_backward (fused)");
  return 0;
}

template <int D, bool CAUSAL, bool SEQ, bool BIAS>
static int launch_flash_backward_three(const bf16_t* q, const bf16_t* k,
                                       const bf16_t* v, const bf16_t* dout,
                                       bf16_t* dq, bf16_t* dk, bf16_t* dv,
                                       const float* lse, const float* delta,
                                       int B, int L, int H, const int32_t* seq,
                                       const float* tab, float* dtab,
                                       hipStream_t st) {
  int rc = launch_flash_backward_one<D, CAUSAL, BWD_DV, SEQ, BIAS>(
      q, k, v, dout, lse, delta, dv, B, L, H, seq, tab, dtab, st);
  if (rc != 0) return rc;
  rc = launch_flash_backward_one<D, CAUSAL, BWD_DK, SEQ, BIAS>(
      q, k, v, dout, lse, delta, dk, B, L, H, seq, tab, dtab, st);
  if (rc != 0) return rc;
  return launch_flash_backward_one<D, CAUSAL, BWD_DQ, SEQ, BIAS>(
      q, k, v, dout, lse, delta, dq, B, L, H, seq, tab, dtab, st);
}

// delta[b * H + h][q] = sum_d dout . out for the rows of [B, L, H * D] tensors:
// 16 lanes per (row, head), 16 bytes per lane and 16-byte step.
template <int D>
__global__ __launch_bounds__(256) void attention_delta_kernel(
    const bf16_t* __restrict__ dout, const bf16_t* __restrict__ out,
    float* __restrict__ delta, int64_t rows_heads, int L, int H) {
  const int64_t item = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  float sum = 0.f;
  if (item < rows_heads) {
    const bf16_t* a = dout + item * D;
    const bf16_t* b = out + item * D;
#pragma unroll
    for (int c = sub * 8; c < D; c += 128) {
      const uint4 x = load_streaming(reinterpret_cast<const uint4*>(a + c));
      const uint4 y = load_streaming(reinterpret_cast<const uint4*>(b + c));
      float fx[8], fy[8];
      unpack16(x, fx, bf16_t());
      unpack16(y, fy, bf16_t());
#pragma unroll
      for (int u = 0; u < 8; ++u) sum = fmaf(fx[u], fy[u], sum);
    }
  }
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) sum += __shfl_xor(sum, off);
  if (item < rows_heads && sub == 0) {
    const int64_t row = item / H;               // b * L + q
    const int h = (int)(item - row * H);
    const int64_t b = row / L, qi = row - b * L;
    delta[(b * H + h) * L + qi] = sum;
  }
}

// lse_saved / out_saved: the forward pass's softmax denominators and outputs
// when the caller kept them; otherwise a pass in the forward kernel's shape
// recomputes the denominators (and delta from the unrounded outputs).
template <int D, bool CAUSAL, bool SEQ, bool BIAS>
static int launch_flash_backward(const bf16_t* q, const bf16_t* k,
                                 const bf16_t* v, const bf16_t* dout,
                                 bf16_t* dq, bf16_t* dk, bf16_t* dv, float* lse,
                                 float* delta, int B, int L, int H,
                                 const int32_t* seq, const float* tab,
                                 float* dtab, const bf16_t* out_saved,
                                 const float* lse_saved, hipStream_t st) {
  using Cfg = FlashCfg<D>;
  if (out_saved != nullptr) {
    const int64_t items = (int64_t)B * L * H;
    attention_delta_kernel<D><<<(unsigned)((items * 16 + 255) / 256), 256, 0,
                                st>>>(dout, out_saved, delta, items, L, H);
    MOE_CHECK_LAUNCH("self_attention_backward (delta)");
  } else {
    constexpr int LDS = Cfg::LDS_BYTES + 512 + 1536;
    dim3 grid((unsigned)((L + Cfg::BQ - 1) / Cfg::BQ), (unsigned)(B * H));
    auto stats = flash_attention_kernel<D, CAUSAL, true, SEQ, BIAS>;
    MOE_ALLOW_LDS(stats, LDS);
    stats<<<grid, Cfg::THREADS, LDS, st>>>(q, k, v, nullptr, L, H, dout, lse,
                                           delta, seq, tab);
    MOE_CHECK_LAUNCH("self_attention_backward (lse, delta)");
  }
  const float* lse_use = out_saved != nullptr ? lse_saved : lse;
  return launch_flash_backward_three<D, CAUSAL, SEQ, BIAS>(
      q, k, v, dout, dq, dk, dv, lse_use, delta, B, L, H, seq, tab, dtab, st);
}

__global__ void fill_zero_kernel(float* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// dvalues[h][b] = sum of dtab[h][d] over the distances d of bucket b (the
// gradient of the gather), rounded to bf16.  One wavefront per (bucket, head):
// lanes stride over the distances, then a butterfly sum.
__global__ __launch_bounds__(64) void relative_table_backward_kernel(
    const float* __restrict__ dtab, const int32_t* __restrict__ bucket,
    bf16_t* __restrict__ dvalues, int n, int NB) {
  const int b = blockIdx.x;
  const float* row = dtab + (int64_t)blockIdx.y * n;
  float sum = 0.f;
  for (int d = threadIdx.x; d < n; d += 64)
    if (bucket[d] == b) sum += row[d];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off);
  if (threadIdx.x == 0)
    store_f32<bf16_t>(dvalues + (int64_t)blockIdx.y * NB + b, sum);
}

size_t flash_attention_backward_workspace_bytes(int B, int L, int H,
                                                bool relative_bias) {
  return 2 * (((size_t)B * H * L * sizeof(float) + 255) & ~(size_t)255) + 256 +
         (relative_bias ? 2 * relative_table_bytes(L, H) : 0);
}

int flash_attention_backward(const void* q, const void* k, const void* v,
                             const void* dout, void* dq, void* dk, void* dv,
                             int B, int L, int H, int D, int causal,
                             const int32_t* sequence_id, const void* rel_values,
                             const int32_t* rel_bucket, int num_buckets,
                             void* dvalues, const void* out_saved,
                             const float* lse_saved, void* workspace,
                             hipStream_t st) {
  const size_t per = (((size_t)B * H * L * sizeof(float) + 255) & ~(size_t)255) /
                     sizeof(float);
  float* lse = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  float* delta = lse + per;
  float *tab = nullptr, *dtab = nullptr;
  const int n = 2 * L - 1;
  if (rel_values != nullptr) {
    tab = delta + per;
    dtab = tab + relative_table_bytes(L, H) / sizeof(float);
    int rc = launch_relative_table(rel_values, rel_bucket, tab, L, H,
                                   num_buckets, st);
    if (rc != 0) return rc;
    const int64_t cells = (int64_t)H * n;
    fill_zero_kernel<<<(unsigned)((cells + 255) / 256), 256, 0, st>>>(dtab, cells);
    MOE_CHECK_LAUNCH("self_attention_backward (clear)");
  }
  const bf16_t *q_ = (const bf16_t*)q, *k_ = (const bf16_t*)k,
               *v_ = (const bf16_t*)v, *d_ = (const bf16_t*)dout;
  bf16_t *dq_ = (bf16_t*)dq, *dk_ = (bf16_t*)dk, *dv_ = (bf16_t*)dv;
  const int rc = flash_dispatch(
      causal != 0, sequence_id != nullptr, tab != nullptr,
      [&](auto c, auto s, auto bi) {
        constexpr bool C = decltype(c)::value, S = decltype(s)::value,
                       BI = decltype(bi)::value;
        if (D == 128)
          return launch_flash_backward<128, C, S, BI>(
              q_, k_, v_, d_, dq_, dk_, dv_, lse, delta, B, L, H, sequence_id,
              tab, dtab, (const bf16_t*)out_saved, lse_saved, st);
        return launch_flash_backward<64, C, S, BI>(
            q_, k_, v_, d_, dq_, dk_, dv_, lse, delta, B, L, H, sequence_id, tab,
            dtab, (const bf16_t*)out_saved, lse_saved, st);
      });
  if (rc != 0 || rel_values == nullptr) return rc;
  relative_table_backward_kernel<<<dim3((unsigned)num_buckets, (unsigned)H), 64,
                                   0, st>>>(dtab, rel_bucket, (bf16_t*)dvalues,
                                            n, num_buckets);
  MOE_CHECK_LAUNCH("self_attention_backward (bias values)");
  return 0;
}

}  // namespace mesh_moe
