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

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void flash_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, bf16_t* __restrict__ out, int L, int H) {
  using Cfg = FlashCfg<D>;
  extern __shared__ __attribute__((aligned(16))) unsigned char fa_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int nq = (L + Cfg::BQ - 1) / Cfg::BQ;
  const int qt = nq - 1 - (int)blockIdx.x;   // long (late) query tiles first
  const int bh = blockIdx.y, b = bh / H, h = bh % H;
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
    const bool need_mask =
        (CAUSAL && key0 + Cfg::BK - 1 > qw_first) || key0 + Cfg::BK > L;
    {
      const unsigned char* ks = fa_smem + buf * Cfg::STAGE;
      const unsigned char* vs = ks + Cfg::K_BYTES;
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
      // mask and row maximum
      if (need_mask) {
        // (the empty asm keeps the compiler from turning the branch into 64
        // selects that every tile would execute)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key0 + sub * 32 + 8 * (r / 4) + 4 * half + (r % 4);
            const bool ok = key < L && (!CAUSAL || key <= my_q);
            if (!ok) acc_s[sub][r] = NEG;
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
      const float mneg = -m_new * LOG2E;
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
#pragma unroll
      for (int dt = 0; dt < Cfg::DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[dt][r] *= alpha;
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
  if (my_q < L) {
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

template <int D>
static int launch_flash(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                        bf16_t* out, int B, int L, int H, int causal,
                        hipStream_t st) {
  using Cfg = FlashCfg<D>;
  dim3 grid((unsigned)((L + Cfg::BQ - 1) / Cfg::BQ), (unsigned)(B * H));
  if (causal) {
    auto kern = flash_attention_kernel<D, true>;
    MOE_ALLOW_LDS(kern, Cfg::LDS_BYTES);
    kern<<<grid, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(q, k, v, out, L, H);
  } else {
    auto kern = flash_attention_kernel<D, false>;
    MOE_ALLOW_LDS(kern, Cfg::LDS_BYTES);
    kern<<<grid, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(q, k, v, out, L, H);
  }
  MOE_CHECK_LAUNCH("self_attention (fused)");
  return 0;
}

bool flash_attention_supported(int L, int H, int D, int dtype, const void* q,
                               const void* k, const void* v, const void* out) {
  return dtype == MESH_MOE_BF16 && (D == 64 || D == 128) && L >= 8 &&
         L % 8 == 0 &&
         (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 ==
          0) && (int64_t)L * H * D < (1LL << 31);
}

size_t flash_attention_workspace_bytes(int B, int L, int H, int D) {
  (void)B; (void)L; (void)H; (void)D;
  return 256;     // the fused kernel needs no scratch
}

int flash_attention(const void* q, const void* k, const void* v, void* out,
                    int B, int L, int H, int D, int causal, void* workspace,
                    hipStream_t st) {
  (void)workspace;
  if (D == 128)
    return launch_flash<128>((const bf16_t*)q, (const bf16_t*)k,
                             (const bf16_t*)v, (bf16_t*)out, B, L, H, causal,
                             st);
  return launch_flash<64>((const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v,
                          (bf16_t*)out, B, L, H, causal, st);
}

}  // namespace mesh_moe
