// Expert feed-forward as a grouped GEMM for gfx950:
//   h[e] = act(expert_in[e] . wi[e]),  y[e] = h[e] . wo[e]
// Replaces layers.dense_product "wi" + layers.dense "wo" of
// mesh_tensorflow/transformer/moe.py:469-486 (hierarchical layer: :765-774).
//
// Both GEMMs are "TN": A [R, K] and the packed weight B [N, K] are
// K-contiguous, C [R, N] = A . B^T.  The bf16 kernel uses
// v_mfma_f32_32x32x16_bf16 with LDS double buffering; float32 and odd shapes
// use a plain FMA tile kernel.
#include <type_traits>

#include "common.h"

namespace mesh_moe {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// ---------------------------------------------------------------------------
// bf16 MFMA kernel.
// Block tile BM x BN, K step BK, 4 wavefronts in a 2 x 2 grid, each owning a
// (BM/2) x (BN/2) sub-tile made of 32 x 32 MFMA tiles.  LDS rows hold BK bf16
// plus 8 bf16 of padding, which makes the 16-byte fragment reads of
// consecutive rows hit disjoint banks.
//
// The weight tile is fed as the MFMA "A" operand and the activation tile as
// "B", i.e. each MFMA produces a 32(n) x 32(m) block of C^T.  Per lane l the
// operands are row/column l%32 with k = 8*(l/32)..+7, and accumulator register
// r holds n = 8*(r/4) + 4*(l/32) + r%4 for m = l%32: four consecutive output
// columns per lane, which the epilogue packs into one 8-byte LDS write.  The
// finished tile is staged in LDS and written out with 16-byte row-contiguous
// stores.
// ---------------------------------------------------------------------------
template <int BM, int BN, int BK>
struct GemmCfg {
  static constexpr int THREADS = 256;
  static constexpr int LDK = BK + 8;  // padded LDS row, in bf16
  static constexpr int WTM = BM / 2, WTN = BN / 2;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int CPR = BK / 8;  // 16-byte chunks per tile row
  static constexpr int A_CHUNKS = BM * CPR / THREADS;
  static constexpr int B_CHUNKS = BN * CPR / THREADS;
  static constexpr int LDC = BN + 4;  // padded row of the staged C tile
  static constexpr size_t LOOP_BYTES = 2ull * (BM + BN) * LDK * sizeof(bf16_t);
  static constexpr size_t EPI_BYTES = (size_t)BM * LDC * sizeof(bf16_t);
  static constexpr size_t LDS_BYTES =
      LOOP_BYTES > EPI_BYTES ? LOOP_BYTES : EPI_BYTES;
};

// relu commutes with the rounding (which keeps the sign; -0 and +0 both end as
// +0), so it is applied to the float32 accumulators
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b, bool relu) {
  if (relu) {
    a = fmaxf(a, 0.f);
    b = fmaxf(b, 0.f);
  }
  return f32x2_to_bf16x2(a, b);
}

template <int BM, int BN, int BK, bool RELU, bool OUT_F32 = false>
__global__ __launch_bounds__(256) void grouped_gemm_bf16_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
    void* __restrict__ Cvoid, int R, int N, int K, int tiles_m, int tiles_n) {
  bf16_t* Cout = reinterpret_cast<bf16_t*>(Cvoid);
  using Cfg = GemmCfg<BM, BN, BK>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* As = reinterpret_cast<bf16_t*>(smem_raw);  // [2][BM][LDK]
  bf16_t* Bs = As + 2 * BM * Cfg::LDK;               // [2][BN][LDK]

  // Workgroups are handed to the 8 XCDs round-robin (block b runs on XCD
  // b % 8) and each XCD has its own L2.  Renumber so that every XCD works on a
  // contiguous range of logical tiles; logical tiles walk the M tiles of one
  // (expert, N tile), so the tiles resident on an XCD at one time share a few
  // weight panels and all of the expert's activation rows through that L2.
  const int nblk = gridDim.x;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int q = nblk >> 3, rmd = nblk & 7;
  const int logical = xcd * q + min(xcd, rmd) + local;
  const int tiles_per_e = tiles_m * tiles_n;
  const int e = logical / tiles_per_e;
  const int rem = logical - e * tiles_per_e;
  const int tn = rem / tiles_m;
  const int tm = rem - tn * tiles_m;
  const int row0 = tm * BM, col0 = tn * BN;
  const bf16_t* Ae = A + (int64_t)e * R * K;
  const bf16_t* Be = B + (int64_t)e * N * K;
  bf16_t* Ce = Cout + (int64_t)e * R * N;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging (rows clamped; the K tail reads zeros)
  uint4 areg[Cfg::A_CHUNKS], breg[Cfg::B_CHUNKS];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < Cfg::A_CHUNKS; ++i) {
      int c = tid + i * Cfg::THREADS;
      int r = c / Cfg::CPR, kc = c % Cfg::CPR;
      int gr = min(row0 + r, R - 1);
      int gk = k0 + kc * 8;
      uint4 v = *reinterpret_cast<const uint4*>(Ae + (int64_t)gr * K + min(gk, K - 8));
      areg[i] = gk < K ? v : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_CHUNKS; ++i) {
      int c = tid + i * Cfg::THREADS;
      int r = c / Cfg::CPR, kc = c % Cfg::CPR;
      int gr = min(col0 + r, N - 1);
      int gk = k0 + kc * 8;
      uint4 v = *reinterpret_cast<const uint4*>(Be + (int64_t)gr * K + min(gk, K - 8));
      breg[i] = gk < K ? v : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&](int buf) {
    bf16_t* as = As + buf * BM * Cfg::LDK;
    bf16_t* bs = Bs + buf * BN * Cfg::LDK;
#pragma unroll
    for (int i = 0; i < Cfg::A_CHUNKS; ++i) {
      int c = tid + i * Cfg::THREADS;
      int r = c / Cfg::CPR, kc = c % Cfg::CPR;
      *reinterpret_cast<uint4*>(as + r * Cfg::LDK + kc * 8) = areg[i];
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_CHUNKS; ++i) {
      int c = tid + i * Cfg::THREADS;
      int r = c / Cfg::CPR, kc = c % Cfg::CPR;
      *reinterpret_cast<uint4*>(bs + r * Cfg::LDK + kc * 8) = breg[i];
    }
  };

  f32x16_t acc[Cfg::TM][Cfg::TN];
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global((kt + 1) * BK);
    const bf16_t* as = As + buf * BM * Cfg::LDK + (wm * Cfg::WTM + frag_row) * Cfg::LDK + frag_k;
    const bf16_t* bs = Bs + buf * BN * Cfg::LDK + (wn * Cfg::WTN + frag_row) * Cfg::LDK + frag_k;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8_t af[Cfg::TM], bfr[Cfg::TN];
#pragma unroll
      for (int i = 0; i < Cfg::TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8_t*>(as + i * 32 * Cfg::LDK + kk * 16);
#pragma unroll
      for (int j = 0; j < Cfg::TN; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8_t*>(bs + j * 32 * Cfg::LDK + kk * 16);
#pragma unroll
      for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }

  const int m_l = lane & 31;
  const int n_l = (lane >> 5) * 4;
  if (OUT_F32) {
    // float32 result (attention logits, which the reference keeps in float32):
    // every lane owns 4 consecutive columns per register group
    float* Cf = reinterpret_cast<float*>(Cvoid) + (int64_t)e * R * N;
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i) {
#pragma unroll
      for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int grow = row0 + wm * Cfg::WTM + i * 32 + m_l;
          const int gcol = col0 + wn * Cfg::WTN + j * 32 + 8 * q + n_l;
          if (grow < R && gcol < N) {
            float4 v = make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1],
                                   acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            if (RELU) {
              v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f);
              v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f);
            }
            *reinterpret_cast<float4*>(Cf + (int64_t)grow * N + gcol) = v;
          }
        }
      }
    }
    return;
  }
  // epilogue: round (and relu), stage the tile in LDS, coalesced stores
  bf16_t* Cs = reinterpret_cast<bf16_t*>(smem_raw);  // [BM][LDC]
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i) {
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = wm * Cfg::WTM + i * 32 + m_l;
        const int col = wn * Cfg::WTN + j * 32 + 8 * q + n_l;
        uint2 v;
        v.x = pack2_bf16(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], RELU);
        v.y = pack2_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], RELU);
        *reinterpret_cast<uint2*>(Cs + row * Cfg::LDC + col) = v;
      }
    }
  }
  __syncthreads();
  constexpr int CPR_C = BN / 8;  // 16-byte chunks per output row
#pragma unroll 4
  for (int c = tid; c < BM * CPR_C; c += Cfg::THREADS) {
    const int r = c / CPR_C, cc = (c % CPR_C) * 8;
    const int grow = row0 + r, gcol = col0 + cc;
    if (grow < R && gcol < N) {
      const uint2* s = reinterpret_cast<const uint2*>(Cs + r * Cfg::LDC + cc);
      uint2 lo = s[0], hi = s[1];
      *reinterpret_cast<uint4*>(Ce + (int64_t)grow * N + gcol) =
          make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
  }
}

// ---------------------------------------------------------------------------
// bf16 MFMA kernel with direct global -> LDS loads and an NS-stage ring.
//
// Same tiling and MFMA operand roles as the kernel above, but the K loop is fed
// by global_load_lds_dwordx4: every lane names its own 16 global bytes and the
// wavefront's 64 x 16 bytes land contiguously in LDS without passing through
// registers.  The loads for K tile kt+NS-1 are issued while tile kt is being
// multiplied; a partial vmcnt wait plus one bare s_barrier per K tile publishes
// the oldest tile.
//
// One load instruction fetches 8 rows x 128 bytes (BK = 64 bf16): 8 consecutive
// lanes read one full 128-byte line of a row, which is what the memory
// pipeline coalesces best (lanes that stride across rows run ~4x slower).
// LDS therefore holds plain 128-byte rows, and bank conflicts are avoided by
// an XOR swizzle of the 16-byte chunk index applied on the GLOBAL side: the
// lane that fills LDS slot (row, p) loads chunk p ^ swz(row), with
// swz(row) = (row & 7) ^ ((row >> 3) & 1).  The MFMA fragment read of 16
// consecutive rows at one chunk then touches 16 distinct 16-byte columns of a
// 256-byte window (and any 8 consecutive rows 8 distinct columns of 128 bytes).
// Requires K % 64 == 0 and per-expert operand sizes below 2^30 elements.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void lds_void_t;
typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt with expcnt / lgkmcnt left at "no wait"
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void lds_write_b64_asm(uint32_t addr, u32x2_t v) {
  asm volatile("ds_write_b64 %0, %1" :: "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ u32x4_t lds_read_b128_asm(uint32_t addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
// Waits for the LDS reads above; the values pass through it so that nothing
// that uses them is scheduled ahead of the wait.
template <int N>
__device__ __forceinline__ void lds_wait_pieces(u32x4_t (&p)[N]) {
  static_assert(N == 8, "eight pieces per pass");
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]), "+v"(p[4]),
                 "+v"(p[5]), "+v"(p[6]), "+v"(p[7])
               :: "memory");
}

// Block barrier that publishes LDS writes and waits for nothing else: vector
// memory loads and stores of this wavefront stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int BM, int BN, int WN, int WM = 2>  // WM x WN wavefronts
struct DmaCfg {
  static constexpr int BK = 64;
  static constexpr int NS = 2;                         // LDS slots
  static constexpr int WAVES = WM * WN;
  static constexpr int THREADS = 64 * WAVES;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int ROW_BYTES = BK * 2;             // 128
  static constexpr int A_INSTR = (BM / 8) / WAVES;     // per wavefront
  static constexpr int B_INSTR = (BN / 8) / WAVES;
  static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDC = BN + 4;
  static constexpr size_t LOOP_BYTES = (size_t)NS * STAGE_BYTES;
  static constexpr size_t EPI_BYTES = (size_t)BM * LDC * sizeof(bf16_t);
  static constexpr size_t LDS_BYTES =
      LOOP_BYTES > EPI_BYTES ? LOOP_BYTES : EPI_BYTES;
};

__device__ __forceinline__ int lds_swizzle(int row) {
  return (row & 7) ^ ((row >> 3) & 1);
}

template <int BM, int BN, int WN, bool RELU, int WM = 2>
__global__ __launch_bounds__(64 * WM * WN) void grouped_gemm_bf16_dma_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
    bf16_t* __restrict__ Cout, int R, int N, int K, int tiles_m, int tiles_n) {
  using Cfg = DmaCfg<BM, BN, WN, WM>;
  constexpr int BK = Cfg::BK;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

  const int nblk = gridDim.x;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int per_xcd = nblk >> 3, extra = nblk & 7;
  const int logical = xcd * per_xcd + min(xcd, extra) + local;
  const int tiles_per_e = tiles_m * tiles_n;
  const int e = logical / tiles_per_e;
  const int rem = logical - e * tiles_per_e;
  const int tn = rem / tiles_m;
  const int tm = rem - tn * tiles_m;
  const int row0 = tm * BM, col0 = tn * BN;
  const bf16_t* Ae = A + (int64_t)e * R * K;
  const bf16_t* Be = B + (int64_t)e * N * K;
  bf16_t* Ce = Cout + (int64_t)e * R * N;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  // Element offsets of the 16 bytes this lane fetches in each of its load
  // instructions.  Instruction q of an operand covers tile rows 8q .. 8q+7;
  // lane l fills LDS slot (row 8q + l/8, column l%8).  Wavefront w issues
  // q = w, w + 4, ...
  int a_off[Cfg::A_INSTR], b_off[Cfg::B_INSTR];
#pragma unroll
  for (int j = 0; j < Cfg::A_INSTR; ++j) {
    const int row = (wave + Cfg::WAVES * j) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ lds_swizzle(row);
    a_off[j] = min(row0 + row, R - 1) * K + chunk * 8;
  }
#pragma unroll
  for (int j = 0; j < Cfg::B_INSTR; ++j) {
    const int row = (wave + Cfg::WAVES * j) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ lds_swizzle(row);
    b_off[j] = min(col0 + row, N - 1) * K + chunk * 8;
  }
  auto issue_stage = [&](int kt, int slot) {
    unsigned char* sa = smem_raw + slot * Cfg::STAGE_BYTES;
    unsigned char* sb = sa + Cfg::A_BYTES;
    const bf16_t* ak = Ae + kt * BK;
    const bf16_t* bk = Be + kt * BK;
#pragma unroll
    for (int j = 0; j < Cfg::A_INSTR; ++j)
      __builtin_amdgcn_global_load_lds(
          (glb_void_t*)(ak + a_off[j]),
          (lds_void_t*)(sa + (wave + Cfg::WAVES * j) * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < Cfg::B_INSTR; ++j)
      __builtin_amdgcn_global_load_lds(
          (glb_void_t*)(bk + b_off[j]),
          (lds_void_t*)(sb + (wave + Cfg::WAVES * j) * 1024), 16, 0, 0);
  };

  f32x16_t acc[Cfg::TM][Cfg::TN];
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Fragment reads: this lane reads row l % 32 of each 32-row MFMA tile of its
  // wavefront's sub-tile, chunk 2*kk + l/32 of the K tile, at the swizzled
  // column.  The swizzle depends only on the low four row bits, which every
  // MFMA tile of the sub-tile shares.
  const int fr = lane & 31, fc = lane >> 5;
  int a_frag[BK / 16], b_frag[BK / 16];
#pragma unroll
  for (int kk = 0; kk < BK / 16; ++kk) {
    const int col = ((kk * 2 + fc) ^ lds_swizzle(fr)) * 16;
    a_frag[kk] = (wm * Cfg::WTM + fr) * Cfg::ROW_BYTES + col;
    b_frag[kk] = (wn * Cfg::WTN + fr) * Cfg::ROW_BYTES + col;
  }

  // K loop, NS = 2 slots.  The MFMA fragments are double buffered in registers:
  // while the 16 MFMAs of step kk run, the 8 fragment reads of step kk+1 are in
  // flight.  The hand-over to the next K tile happens before the MFMAs of the
  // LAST step of a tile: once this lane holds that step's fragments it no
  // longer needs the tile's LDS slot, so it waits for its own loads of the next
  // tile, meets the other wavefronts at a bare s_barrier (__syncthreads() would
  // add a fence that also drains the loads that are meant to stay in flight),
  // issues the loads of tile kt+2 into the slot just freed and reads the first
  // fragments of tile kt+1 -- all of it hidden behind the last 16 MFMAs.
  constexpr int KSTEPS = BK / 16;
  const int nk = K / BK;
  bf16x8_t fa[2][Cfg::TM], fb[2][Cfg::TN];
  auto read_frags = [&](int slot, int kk, int buf) {
    const unsigned char* sa = smem_raw + slot * Cfg::STAGE_BYTES;
    const unsigned char* sb = sa + Cfg::A_BYTES;
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i)
      fa[buf][i] = *reinterpret_cast<const bf16x8_t*>(sa + a_frag[kk] + i * 32 * Cfg::ROW_BYTES);
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j)
      fb[buf][j] = *reinterpret_cast<const bf16x8_t*>(sb + b_frag[kk] + j * 32 * Cfg::ROW_BYTES);
  };

  issue_stage(0, 0);
  wait_vmcnt<0>();
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (nk > 1) issue_stage(1, 1);
  read_frags(0, 0, 0);
  // One K tile.  LAST = the final tile (no hand-over).  The body is free of
  // branches so that the scheduling hints below see one basic block; past the
  // end of K the hand-over simply re-fetches the last tile into the free slot.
  auto k_tile = [&](int kt, auto last_tag) {
    constexpr bool LAST = decltype(last_tag)::value;
    const int slot = kt & 1;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      if (kk + 1 < KSTEPS) {
        read_frags(slot, kk + 1, nxt);
      } else if (!LAST) {
        // fragments of the last step are in registers (lgkmcnt 0) and this
        // lane's loads of tile kt+1 have landed (vmcnt 0)
        __builtin_amdgcn_s_waitcnt(0x0070);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_stage(min(kt + 2, nk - 1), slot);
        read_frags(slot ^ 1, 0, nxt);
      }
#pragma unroll
      for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
      // Spread the memory instructions of this step between its MFMAs instead
      // of letting them queue up in front (masks: 0x8 MFMA, 0x20 VMEM read,
      // 0x100 LDS read).
      constexpr int READS = Cfg::TM + Cfg::TN;
      constexpr int MFMA_PER_READ = Cfg::TM * Cfg::TN / READS;
      constexpr int LOADS = Cfg::A_INSTR + Cfg::B_INSTR;
      if (kk + 1 < KSTEPS) {
#pragma unroll
        for (int g = 0; g < READS; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, MFMA_PER_READ, 0);
        }
      } else if (!LAST) {
#pragma unroll
        for (int g = 0; g < READS; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, (LOADS + READS - 1) / READS, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
      }
    }
  };
  for (int kt = 0; kt + 1 < nk; ++kt) k_tile(kt, std::false_type{});
  k_tile(nk - 1, std::true_type{});
  // the epilogue reuses the ring: no direct-to-LDS load may still be in flight
  // (the last hand-over re-fetches a tile nobody reads)
  wait_vmcnt<0>();
  __syncthreads();

  // epilogue: round (and relu), stage the tile in LDS, coalesced stores
  bf16_t* Cs = reinterpret_cast<bf16_t*>(smem_raw);  // [BM][LDC]
  const int m_l = lane & 31;
  const int n_l = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i) {
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = wm * Cfg::WTM + i * 32 + m_l;
        const int col = wn * Cfg::WTN + j * 32 + 8 * q + n_l;
        uint2 v;
        v.x = pack2_bf16(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], RELU);
        v.y = pack2_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], RELU);
        *reinterpret_cast<uint2*>(Cs + row * Cfg::LDC + col) = v;
      }
    }
  }
  __syncthreads();
  constexpr int CPR_C = BN / 8;  // 16-byte chunks per output row
#pragma unroll 4
  for (int c = tid; c < BM * CPR_C; c += Cfg::THREADS) {
    const int r = c / CPR_C, cc = (c % CPR_C) * 8;
    const int grow = row0 + r, gcol = col0 + cc;
    if (grow < R && gcol < N) {
      const uint2* s = reinterpret_cast<const uint2*>(Cs + r * Cfg::LDC + cc);
      uint2 lo = s[0], hi = s[1];
      *reinterpret_cast<uint4*>(Ce + (int64_t)grow * N + gcol) =
          make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
  }
}

// ---------------------------------------------------------------------------
// bf16 MFMA kernel for 256 x 256 tiles with SPREAD direct-to-LDS loads.
//
// Same tile, wavefront grid (2 x 4, 128 x 64 sub-tiles), LDS image and
// fragment reads as grouped_gemm_bf16_dma_kernel<256, 256, 4, RELU, 2>; the
// difference is when the loads are issued.  A wavefront that issues its eight
// loads of a K tile back to back sits in that burst for ~0.7 us (the memory
// pipeline accepts them only as fast as earlier requests drain), and because
// the wavefronts of a block hand over together, the MFMA pipes idle meanwhile.
// Here the 160 KB of LDS hold two slots for the token tile and THREE for the
// weight tile, which lets the loads of tile t+2 ride on the MFMA steps of
// tile t, pinned between its MFMAs:
//
//   step 0:            weight loads 0,1 of tile t+2   (two tiles ahead)
//   step 1, step 2:    weight load 2 / weight load 3 of tile t+2
//   step 3 (after the hand-over barrier that frees their slot, behind the
//           first fragment reads of tile t+1): the four token loads of tile t+2
//
// vmcnt counts in issue order, so the hand-over of tile t waits with vmcnt(4):
// everything up to the token loads of tile t+1 has landed, the four weight
// loads of tile t+2 stay in flight.
// ---------------------------------------------------------------------------
// Two ds_read_b64_tr_b16 at byte offsets OFF and OFF + 2048 from LDS address
// `addr` (see the K-major variant of the ring kernel).
template <int OFF>
__device__ __forceinline__ void lds_read_tr16_pair(uint32_t addr, i16x4_t& lo,
                                                   i16x4_t& hi) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(lo) : "v"(addr), "n"(OFF));
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(hi) : "v"(addr), "n"(OFF + 2048));
}

struct RingCfg {
  static constexpr int BM = 256, BN = 256, BK = 64, WM = 2, WN = 4;
  static constexpr int WAVES = WM * WN, THREADS = 64 * WAVES;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int ROW_BYTES = BK * 2;
  static constexpr int A_INSTR = (BM / 8) / WAVES, B_INSTR = (BN / 8) / WAVES;
  static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
  static constexpr int A_SLOTS = 2, B_SLOTS = 3;
  static constexpr int B_BASE = A_SLOTS * A_BYTES;
  static constexpr size_t LOOP_BYTES = (size_t)A_SLOTS * A_BYTES + (size_t)B_SLOTS * B_BYTES;
  static constexpr size_t LDS_BYTES = LOOP_BYTES;  // the epilogue stages inside
  static_assert(A_INSTR == 4 && B_INSTR == 4, "load schedule assumes 4 + 4");
};

// GATHER: the rows of expert e's first operand are not A[e][r] but rows of a
// shared token matrix, A[row_map[e * R + r]] (row_map < 0: the all-zero row
// `zero_row`): the dispatch of the Mixture-of-Experts layer folded into the
// first expert GEMM's loads.
//
// KMAJOR: both operands are stored with the reduction index outermost,
// A[e][k][r] and B[e][k][n] (C = A^T . B, the weight gradients of the expert
// einsums: the reduction runs over token rows).  A K tile is then 64 rows of
// 256 consecutive elements; it goes to LDS as it lies in memory (row k at byte
// 512 k, the 64-byte units of a row XOR-ed with k % 4 against bank
// conflicts) and the MFMA operands, which need 8 consecutive k per lane, are
// read with ds_read_b64_tr_b16: within 16 lanes, lane t addresses the 8 bytes
// at (row t / 4, elements 4 (t % 4) ..) of a 4 x 16 block and lane i receives
// the block's column i.  R, N multiples of 8.  With k_extent, expert e's
// reduction stops after its first k_extent[e] rows, rounded up to a K tile
// (rows up to there must hold finite values in one operand and zeros in the
// other); k_extent[e] == 0 gives an all-zero result.  K need not be a
// multiple of the K tile: the rows of the last tile past K come from a zero
// buffer.
//
// MASKED: element (e, r, n) of the result is stored as zero unless
// mask_src[e][r][n] > 0 (the backward of a ReLU whose output is mask_src,
// applied while the tile is written out).  The elements that stay are
// multiplied by mask_scale and rounded again (the backward of a dropout in
// front of the ReLU's consumer: where the stored activation is positive the
// element was kept, and its noise is 1 / keep_prob).
//
// LISTED: only the tiles named in tile_list[0 .. tile_list[-1]) are computed
// (logical tile numbers in ascending order, their count in the element before
// the list): an expert whose occupied rows were moved to the front of its row
// range needs no tiles for the rest (see mesh_moe_compact_expert_ffn).
// (Skipping, inside an expert's last listed tile, the 32-row pieces of a
// wavefront's sub-tile that lie past the occupied rows -- about a tenth of the
// multiply-adds with 1024 +- 32 rows per expert -- made the launches 2 to 5 %
// slower; so did letting only the wavefronts of a tile's empty second half
// skip their multiply-adds, with the flag carried in the list entry: 5 %
// slower, although nothing was added to the path of the full tiles but a
// second copy of the K loop next to it.)
//
// TAILS (R not a multiple of the 256-row tile): in an expert's last row tile
// a wavefront multiplies only the 32-row pieces of its 128-row sub-tile that
// hold rows below R -- the piece count is the same for the whole K loop, so
// the wavefront runs the copy of the loop written for that count (0 to 4
// pieces; with 0 it only loads and meets the barriers).  The two wavefronts of
// a SIMD own the upper and the lower half of the tile, so a tile with 144
// valid rows costs the SIMD 4 + 1 pieces instead of 8.  (Numbering the
// experts' last row tiles after all full ones, so that the persistent blocks
// end on the cheaper tiles, separates the row tiles that share a weight panel:
// with 400 rows per expert the weights were then read twice from memory and
// the launches took 14 % longer; moving only as many last row tiles as the
// final, partly filled round holds to the end cost 5 % where it applied, 640
// rows per expert with 384 tiles, for the same reason.)
// 512 bytes that stay zero (nothing writes them): where a K-major tile reaches
// past the last reduction row, its rows are loaded from here
static __device__ __attribute__((aligned(256))) bf16_t kmajor_zero_row[256];

template <bool RELU, bool GATHER = false, bool KMAJOR = false,
          bool MASKED = false, bool LISTED = false, bool TAILS = false>
__global__ __launch_bounds__(RingCfg::THREADS) void grouped_gemm_bf16_ring_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
    bf16_t* __restrict__ Cout, int R, int N, int K, int tiles_m, int tiles_n,
    int total_tiles, const int32_t* __restrict__ row_map = nullptr,
    const bf16_t* __restrict__ zero_row = nullptr,
    const bf16_t* __restrict__ mask_src = nullptr,
    const int32_t* __restrict__ tile_list = nullptr,
    const int32_t* __restrict__ row_count = nullptr,
    float mask_scale = 1.0f) {
  using Cfg = RingCfg;
  // row_count [E], optional: KMAJOR kernels take it as the reduction extent
  // per expert (k_extent)
  const int32_t* k_extent = KMAJOR ? row_count : nullptr;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, WN = Cfg::WN;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];

  // PERSISTENT blocks: one per CU, each walks a strided list of tiles, so that
  // block start-up and the first loads of a tile overlap the previous tile's
  // epilogue.  Block b runs on XCD b % 8.  The P = blocks / 8 blocks of an XCD
  // hold P consecutive logical tiles at any moment (shared panels in its L2),
  // and consecutive groups of P tiles go to consecutive XCDs: the whole chip
  // then works on the same one or two experts, whose token panels every XCD
  // re-reads from the memory-side cache, instead of on eight experts at once
  // (1 % faster than giving each XCD a contiguous eighth of the tiles).
  const int nblk = gridDim.x;
  if constexpr (LISTED) total_tiles = tile_list[-1];
  int tile, tile_end, tile_step;
  // TAILS: in its round k a block takes the tile k places further (cyclically)
  // among its XCD's P tiles of the round, so that it meets every row tile of
  // the experts in turn, full and partly empty ones: with a fixed place and an
  // even number of row tiles half of the blocks would only ever get the cheap
  // last row tiles and run ahead of the blocks they share weight panels with.
  int round = 0;
  const int xcd_tiles = (nblk & 7) == 0 ? (nblk >> 3) : 0;
  const int xcd_first = (blockIdx.x & 7) * xcd_tiles;
  const int xcd_local = blockIdx.x >> 3;
  auto tile_of_round = [&](int k) {
    const int place = xcd_local + k;
    return k * nblk + xcd_first + (place >= xcd_tiles ? place % xcd_tiles : place);
  };
  if ((nblk & 7) == 0) {
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    tile = xcd * (nblk >> 3) + local;
    tile_end = total_tiles;
    tile_step = nblk;
  } else {
    tile = blockIdx.x;
    tile_end = total_tiles;
    tile_step = nblk;
  }
  if (tile >= tile_end) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int tiles_per_e = tiles_m * tiles_n;
  // K tiles of the current tile's reduction: all of K, or with k_extent
  // (KMAJOR) the expert's first k_extent[e] reduction rows only
  int nk = KMAJOR ? (K + BK - 1) / BK : K / BK;
  bool tile_empty = false;   // k_extent[e] == 0: the result is zero

  // per-tile state
  int row0, col0;
  const bf16_t *Ae, *Be;
  bf16_t* Ce;
  typename std::conditional<GATHER, int64_t, int>::type a_off[Cfg::A_INSTR];
  int b_off[Cfg::B_INSTR];
  // TAILS: 32-row pieces of this wavefront's sub-tile that hold rows below R
  int pieces = Cfg::TM;
  // logical tile -> expert, row tile, column tile
  auto tile_coords = [&](int logical, int& e, int& tm, int& tn) {
    if constexpr (LISTED) logical = tile_list[logical];
    e = logical / tiles_per_e;
    const int rem = logical - e * tiles_per_e;
    tn = rem / tiles_m;
    tm = rem - tn * tiles_m;
    if (!LISTED && !TAILS && tiles_m > 8 && (tiles_m & 7) == 0 &&
        (tiles_n & 3) == 0) {
      // 32 consecutive logical tiles (what an XCD holds at any moment) form a
      // block of 8 row tiles x 4 column tiles: 12 operand panels for 32 tiles.
      // With the plain order and many row tiles they would be 32 row tiles of
      // one column tile: 33 panels, every row panel fetched once per column
      // tile.  Blocks follow each other along N, so the next 32 tiles share
      // the 8 row panels.  (8 row tiles: both orders are the same.)
      const int sup = rem >> 5, within = rem & 31;
      const int per_row = tiles_n >> 2;
      const int sm = sup / per_row, sn = sup - sm * per_row;
      tm = sm * 8 + (within & 7);
      tn = sn * 4 + (within >> 3);
    }
  };
  // GATHER: the slot -> token map entries of the four rows this lane loads in
  // a tile.  fetch_map issues the four loads back to back without waiting
  // (written as asm: the compiler would wait for each before issuing the
  // next, four round trips per tile); the caller waits with vmcnt(0) before
  // set_tile of the same tile reads map_src.
  int map_src[Cfg::A_INSTR];
  auto fetch_map = [&](int logical) {
    if constexpr (GATHER) {
      int e, tm, tn;
      tile_coords(logical, e, tm, tn);
#pragma unroll
      for (int j = 0; j < Cfg::A_INSTR; ++j) {
        const int row = (wave + Cfg::WAVES * j) * 8 + (lane >> 3);
        const int32_t* p = row_map + ((int64_t)e * R + min(tm * BM + row, R - 1));
        asm volatile("global_load_dword %0, %1, off"
                     : "=&v"(map_src[j]) : "v"(p) : "memory");
      }
    }
  };
  auto set_tile = [&](int logical) {
    int e, tm, tn;
    tile_coords(logical, e, tm, tn);
    if constexpr (TAILS) {
      const int valid = min(BM, R - tm * BM);
      const int blocks = (valid + 31) >> 5;
      pieces = __builtin_amdgcn_readfirstlane(
          wm == 0 ? min(blocks, Cfg::TM) : max(blocks - Cfg::TM, 0));
    }
    row0 = tm * BM;
    col0 = tn * BN;
    if constexpr (KMAJOR) {
      if (k_extent != nullptr) {
        const int used = k_extent[e];
        tile_empty = used == 0;
        nk = max(1, min((K + BK - 1) / BK, (used + BK - 1) / BK));
      }
    }
    Ae = GATHER ? A : A + (int64_t)e * R * K;
    Be = B + (int64_t)e * N * K;
    Ce = Cout + (int64_t)e * R * N;
#pragma unroll
    for (int j = 0; j < Cfg::A_INSTR; ++j) {
      if constexpr (KMAJOR) {
        // instruction q = wave + WAVES * j fills tile rows 2q and 2q + 1; lane
        // l fills 16-byte position l % 32 of its row with the chunk that
        // belongs there under the unit swizzle
        const int krow = (wave + Cfg::WAVES * j) * 2 + (lane >> 5);
        const int p = lane & 31;
        const int chunk = ((((p >> 2) ^ (krow & 3)) << 2) | (p & 3)) * 8;
        a_off[j] = krow * R + min(row0 + chunk, R - 8);
        b_off[j] = krow * N + min(col0 + chunk, N - 8);
        continue;
      }
      const int row = (wave + Cfg::WAVES * j) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swizzle(row);
      if constexpr (GATHER) {
        const int src = map_src[j];
        a_off[j] = (src >= 0 ? (int64_t)src * K : (int64_t)(zero_row - A)) +
                   chunk * 8;
      } else {
        a_off[j] = min(row0 + row, R - 1) * K + chunk * 8;
      }
      b_off[j] = min(col0 + row, N - 1) * K + chunk * 8;
    }
  };
  // load j of the token (A, two slots at LDS offset 0) / weight (B, three
  // slots behind them) tile kt; kt past the end re-fetches the last tile into
  // a slot nobody reads any more
  constexpr int B_BASE = Cfg::B_BASE;
  // KMAJOR: load j of a tile fills reduction rows 2 (wave + WAVES j) and + 1
  // (lanes 32-63) of it; past the last reduction row they are zeros
  auto kmajor_past_end = [&](int kt, int j) {
    return kt * BK + (wave + Cfg::WAVES * j) * 2 + (lane >> 5) >= K;
  };
  auto load_a = [&](int kt, int j) {
    const int slot = kt & 1;
    kt = min(kt, nk - 1);
    const bf16_t* src = Ae + kt * (KMAJOR ? BK * R : BK) + a_off[j];
    if constexpr (KMAJOR) {
      if (kmajor_past_end(kt, j)) src = kmajor_zero_row + (lane & 31) * 8;
    }
    __builtin_amdgcn_global_load_lds(
        (glb_void_t*)src,
        (lds_void_t*)(smem_raw + slot * Cfg::A_BYTES +
                      (wave + Cfg::WAVES * j) * 1024), 16, 0, 0);
  };
  auto load_b = [&](int kt, int slot, int j) {
    kt = min(kt, nk - 1);
    const bf16_t* src = Be + kt * (KMAJOR ? BK * N : BK) + b_off[j];
    if constexpr (KMAJOR) {
      if (kmajor_past_end(kt, j)) src = kmajor_zero_row + (lane & 31) * 8;
    }
    __builtin_amdgcn_global_load_lds(
        (glb_void_t*)src,
        (lds_void_t*)(smem_raw + B_BASE + slot * Cfg::B_BYTES +
                      (wave + Cfg::WAVES * j) * 1024), 16, 0, 0);
  };
  // the first loads of a tile except weight tile 1, whose slot the epilogue of
  // the previous tile still uses as staging area
  auto prologue_head = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) load_a(0, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) load_b(0, 0, j);
  };
  auto prologue_tail = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) load_b(1, 1, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) load_a(1, j);
  };

  f32x16_t acc[Cfg::TM][Cfg::TN];

  const int fr = lane & 31, fc = lane >> 5;
  int a_frag[BK / 16], b_frag[BK / 16];
  if constexpr (KMAJOR) {
    // byte offset of this lane's 8 bytes for 32-column block n of its
    // wavefront's sub-tile, at step 0 / first half: a_frag[n], b_frag[n]
    static_assert(Cfg::TM <= BK / 16 && Cfg::TN <= BK / 16, "offset arrays");
    const int t = lane & 15, g = lane >> 4;
    const int inner = ((g & 1) * 16 + 4 * (t & 3)) * 2 +
                      ((g >> 1) * 8 + (t >> 2)) * 512;
#pragma unroll
    for (int n = 0; n < Cfg::TM; ++n)
      a_frag[n] = (((wm * Cfg::TM + n) ^ (t >> 2)) * 64) + inner;
#pragma unroll
    for (int n = 0; n < Cfg::TN; ++n)
      b_frag[n] = (((wn * Cfg::TN + n) ^ (t >> 2)) * 64) + inner;
  } else {
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int col = ((kk * 2 + fc) ^ lds_swizzle(fr)) * 16;
      a_frag[kk] = (wm * Cfg::WTM + fr) * Cfg::ROW_BYTES + col;
      b_frag[kk] = (wn * Cfg::WTN + fr) * Cfg::ROW_BYTES + col;
    }
  }
  constexpr int KSTEPS = BK / 16;
  bf16x8_t fa[2][Cfg::TM], fb[2][Cfg::TN];
  // 8 consecutive k of one column of a K-major tile: two transposed reads at
  // LDS byte address `at` + 8192 kk (+ 2048 for the second four).  Written as
  // asm because the compiler puts a vmcnt(0) in front of the builtin form (it
  // takes the read for a possible LDS store racing the direct-to-LDS loads),
  // which would drain the loads that are meant to stay in flight.  The
  // compiler therefore does not know when the data arrives: wait_frags()
  // (lgkmcnt(0)) stands before the MFMAs that use it.
  const uint32_t lds0 = (uint32_t)(size_t)(lds_void_t*)smem_raw;
  auto read_tr = [&](uint32_t at, int kk) {
    i16x4_t lo, hi;
    switch (kk) {
      case 0: lds_read_tr16_pair<0>(at, lo, hi); break;
      case 1: lds_read_tr16_pair<8192>(at, lo, hi); break;
      case 2: lds_read_tr16_pair<16384>(at, lo, hi); break;
      default: lds_read_tr16_pair<24576>(at, lo, hi); break;
    }
    return __builtin_bit_cast(
        bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto wait_frags = [&]() {
    if constexpr (KMAJOR) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0) only
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // fragment read n of a step: 0..TM-1 token rows, TM..TM+TN-1 weight rows
  auto read_frag = [&](int aslot, int bslot, int kk, int buf, int n) {
    if constexpr (KMAJOR) {
      if (n < Cfg::TM)
        fa[buf][n] = read_tr(lds0 + aslot * Cfg::A_BYTES + a_frag[n], kk);
      else
        fb[buf][n - Cfg::TM] = read_tr(
            lds0 + B_BASE + bslot * Cfg::B_BYTES + b_frag[n - Cfg::TM], kk);
      return;
    }
    if (n < Cfg::TM)
      fa[buf][n] = *reinterpret_cast<const bf16x8_t*>(
          smem_raw + aslot * Cfg::A_BYTES + a_frag[kk] + n * 32 * Cfg::ROW_BYTES);
    else
      fb[buf][n - Cfg::TM] = *reinterpret_cast<const bf16x8_t*>(
          smem_raw + B_BASE + bslot * Cfg::B_BYTES + b_frag[kk] +
          (n - Cfg::TM) * 32 * Cfg::ROW_BYTES);
  };
  auto mfma = [&](int buf, int n) {
    const int i = n / Cfg::TN, j = n % Cfg::TN;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i],
                                                        acc[i][j], 0, 0, 0);
  };
  // with NA of the wavefront's TM row pieces in use: is fragment read n /
  // MFMA n of a step needed?
  auto frag_used = [](int na, int n) {
    return na > 0 && (n >= Cfg::TM || n < na);
  };
  auto mfma_used = [](int na, int n) { return n / Cfg::TN < na; };
  // nothing moves across: the instruction order below is the issue order
  auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
  // fragment reads in the order the MFMAs (token tile i = n / TN outer, weight
  // tile j = n % TN inner) first need them: a0 b0 b1 a1 a2 a3
  constexpr int RD[6] = {0, Cfg::TM, Cfg::TM + 1, 1, 2, 3};

  // bslot = kt % 3, kept incrementally
  int bslot = 0;
  auto k_tile = [&](int kt, auto last_tag, auto na_tag) {
    constexpr bool LAST = decltype(last_tag)::value;
    constexpr int NA = decltype(na_tag)::value;      // row pieces in use
    auto rd = [&](int as, int bs, int kk, int buf, int n) {
      if (frag_used(NA, n)) read_frag(as, bs, kk, buf, n);
    };
    auto mm = [&](int buf, int n) {
      if (mfma_used(NA, n)) mfma(buf, n);
    };
    const int aslot = kt & 1;
    const int bnext = bslot == 2 ? 0 : bslot + 1;       // slot of tile kt+1
    const int bnext2 = bnext == 2 ? 0 : bnext + 1;      // slot of tile kt+2
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      // The loads a step carries: the four weight loads of tile kt+2 over
      // steps 0..2, all four token loads of tile kt+2 right behind the
      // hand-over barrier that frees their slot (a full K tile ahead of use).
      auto load = [&](int which) {
        if (LAST) return;
        if (kk == 0) load_b(kt + 2, bnext2, which);
        if (kk == 1 && which == 0) load_b(kt + 2, bnext2, 2);
        if (kk == 2 && which == 0) load_b(kt + 2, bnext2, 3);
        if (kk == 3) load_a(kt + 2, which);
      };
      if (kk + 1 < KSTEPS) {
        // 6 fragment reads of step kk+1 (in the order its MFMAs need them),
        // 2 loads, 8 MFMAs of step kk
        fence();
        wait_frags();
        rd(aslot, bslot, kk + 1, nxt, RD[0]);
        rd(aslot, bslot, kk + 1, nxt, RD[1]);
        mm(cur, 0); fence();
        rd(aslot, bslot, kk + 1, nxt, RD[2]);
        mm(cur, 1); fence();
        load(0);
        mm(cur, 2); fence();
        rd(aslot, bslot, kk + 1, nxt, RD[3]);
        mm(cur, 3); fence();
        rd(aslot, bslot, kk + 1, nxt, RD[4]);
        mm(cur, 4); fence();
        load(1);
        mm(cur, 5); fence();
        rd(aslot, bslot, kk + 1, nxt, RD[5]);
        mm(cur, 6); fence();
        mm(cur, 7); fence();
      } else if (!LAST) {
        // this lane holds the last step's fragments (lgkmcnt 0); everything
        // but the four weight loads of tile kt+2 has landed (vmcnt 4)
        fence();
        __builtin_amdgcn_s_waitcnt((4 & 15) | (0 << 8) | (7 << 4));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        fence();
        // fragment reads first: a load right behind the barrier would queue
        // up with the other wavefronts' and hold this one's MFMAs back
#pragma unroll
        for (int n = 0; n < 6; ++n) {
          rd(aslot ^ 1, bnext, 0, nxt, RD[n]);
          if (n >= 2) load(n - 2);
          mm(cur, n); fence();
        }
        mm(cur, 6); fence();
        mm(cur, 7); fence();
      } else {
        wait_frags();
#pragma unroll
        for (int n = 0; n < 8; ++n) mm(cur, n);
      }
    }
    bslot = bnext;
  };

  // Epilogue staging: two passes of 128 output rows (64 from each half of the
  // tile, so that all eight wavefronts write), exactly the last two weight
  // slots, which are free once the K loop is over.  Rows are 512 bytes, a
  // multiple of the bank count, so 16-byte chunk c of staging row r lives at
  // chunk c ^ (r & 31): the writes of a wavefront (32 rows x 8 bytes, twice)
  // and its reads (2 rows x 32 chunks) both spread over all banks.
  constexpr int EPI_ROWS = 128;
  constexpr int EPI_ROW_BYTES = BN * 2;
  constexpr int EPI_BASE = B_BASE + Cfg::B_BYTES;
  static_assert(EPI_BASE + EPI_ROWS * EPI_ROW_BYTES <= (int)Cfg::LOOP_BYTES,
                "epilogue staging exceeds the ring");
  static_assert(BN == 256 && Cfg::WM == 2 && Cfg::TM == 4, "epilogue layout");
  // (LDS byte address of the staging area: its accesses are written as asm)
  const uint32_t cs0 = (uint32_t)(size_t)(lds_void_t*)smem_raw + EPI_BASE;
  const int m_l = lane & 31;
  const int half = lane >> 5;   // which 8 bytes of a 16-byte chunk
  constexpr int CPR_C = BN / 8;  // 16-byte chunks per output row

  fetch_map(tile);
  if constexpr (GATHER) {
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
  }
  set_tile(tile);
  prologue_head();
  prologue_tail();
  for (;;) {
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    // K tile 0 has landed: only tile 1 (4 + 4 loads) may still be in flight
    wait_vmcnt<8>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    auto k_loop = [&](auto na_tag) {
      constexpr int NA = decltype(na_tag)::value;
#pragma unroll
      for (int n = 0; n < 6; ++n)
        if (frag_used(NA, RD[n])) read_frag(0, 0, 0, 0, RD[n]);
      bslot = 0;
      for (int kt = 0; kt + 1 < nk; ++kt) k_tile(kt, std::false_type{}, na_tag);
      k_tile(nk - 1, std::true_type{}, na_tag);
    };
    if constexpr (TAILS) {
      switch (pieces) {
        case 0: k_loop(std::integral_constant<int, 0>{}); break;
        case 1: k_loop(std::integral_constant<int, 1>{}); break;
        case 2: k_loop(std::integral_constant<int, 2>{}); break;
        case 3: k_loop(std::integral_constant<int, 3>{}); break;
        default: k_loop(std::integral_constant<int, Cfg::TM>{}); break;
      }
    } else {
      k_loop(std::integral_constant<int, Cfg::TM>{});
    }

    const int next = (TAILS && xcd_tiles != 0) ? tile_of_round(round + 1)
                                               : tile + tile_step;
    const bool has_next = next < tile_end;
    // (the next tile's map entries travel while the ring drains)
    if (has_next) fetch_map(next);
    // Every wavefront is done with the ring and no direct-to-LDS load is in
    // flight (the last hand-over re-fetched a tile nobody reads).
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __syncthreads();
    const int out_row0 = row0, out_col0 = col0;
    bf16_t* out_c = Ce;
    if constexpr (KMAJOR) {
      // an expert without reduction rows: its one K tile held rows that
      // nobody wrote
      if (tile_empty) {
#pragma unroll
        for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
          for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
      }
    }
    if (has_next) {
      // the next tile's first loads fly while this tile is written out
      set_tile(next);
      prologue_head();
    }
    // round (and relu), stage in LDS, coalesced 16-byte stores.  Nothing here
    // waits for vector memory: the next tile's first loads and this tile's
    // stores stay in flight.  (__syncthreads() waits for them at every
    // barrier, and in front of an ordinary LDS access the compiler waits for
    // the direct-to-LDS loads in flight, which might write the same LDS: the
    // staging accesses are therefore asm.)
    // (the staging addresses are formed from a copy of the thread index that
    // the compiler cannot see through: computed once outside the tile loop
    // they would be live across the K loop, which has no registers to spare)
    int e_tid = tid;
    asm volatile("" : "+v"(e_tid));
    const int e_lane = e_tid & 63, e_wave = e_tid >> 6;
    const int e_wm = e_wave / WN, e_wn = e_wave % WN;
    const int e_ml = e_lane & 31, e_half = e_lane >> 5;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int i = pass * 2 + ii;
        const int srow = e_wm * 64 + ii * 32 + e_ml;
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int chunk = (e_wn * Cfg::WTN + j * 32 + 8 * q) / 8;
            u32x2_t v;
            v.x = pack2_bf16(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], RELU);
            v.y = pack2_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3], RELU);
            lds_write_b64_asm(cs0 + srow * EPI_ROW_BYTES +
                                  ((chunk ^ e_ml) * 16) + e_half * 8, v);
          }
        }
      }
      lds_barrier();
      // all staged pieces of this pass first, one wait, then the stores
      constexpr int PIECES = EPI_ROWS * CPR_C / Cfg::THREADS;
      static_assert(EPI_ROWS * CPR_C % Cfg::THREADS == 0, "whole pieces");
      u32x4_t piece[PIECES];
#pragma unroll
      for (int n = 0; n < PIECES; ++n) {
        const int c = e_tid + n * Cfg::THREADS;
        const int srow = c / CPR_C, chunk = c % CPR_C;
        piece[n] = lds_read_b128_asm(cs0 + srow * EPI_ROW_BYTES +
                                     ((chunk ^ (srow & 31)) * 16));
      }
      lds_wait_pieces(piece);
#pragma unroll
      for (int n = 0; n < PIECES; ++n) {
        const int c = e_tid + n * Cfg::THREADS;
        const int srow = c / CPR_C, chunk = c % CPR_C;
        // staging row -> tile row: 64 rows of each half of the tile
        const int grow = out_row0 + (srow >> 6) * 128 + pass * 64 + (srow & 63);
        const int gcol = out_col0 + chunk * 8;
        if (grow < R && gcol < N) {
          u32x4_t v = piece[n];
          if constexpr (MASKED) {
            const u32x4_t hm = *reinterpret_cast<const u32x4_t*>(
                mask_src + (out_c - Cout) + (int64_t)grow * N + gcol);
            if (mask_scale != 1.0f) {
#pragma unroll
              for (int q = 0; q < 4; ++q)
                v[q] = f32x2_to_bf16x2(
                    __builtin_bit_cast(float, v[q] << 16) * mask_scale,
                    __builtin_bit_cast(float, v[q] & 0xffff0000u) * mask_scale);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t keep =
                  (__builtin_bit_cast(float, hm[q] << 16) > 0.f ? 0xffffu : 0u) |
                  (__builtin_bit_cast(float, hm[q] & 0xffff0000u) > 0.f
                       ? 0xffff0000u : 0u);
              v[q] &= keep;
            }
          }
          *reinterpret_cast<u32x4_t*>(out_c + (int64_t)grow * N + gcol) = v;
        }
      }
      lds_barrier();
    }
    if (!has_next) break;
    tile = next;
    ++round;
    prologue_tail();   // the staging area is free again
  }
}

// ---------------------------------------------------------------------------
// float32 on the matrix cores: v_mfma_f32_32x32x2_f32, true float32 operands
// and accumulation (the float32 configuration of the layer: no narrowing).
// Block tile 128 x 128, K step 32, 4 wavefronts in a 2 x 2 grid, each a 64 x 64
// sub-tile = 2 x 2 MFMA tiles.  As in the bf16 kernels the weight tile is the
// MFMA's first operand, so a lane ends up with 4 consecutive output columns
// per register group.  One MFMA consumes k = 2 s + (lane / 32) for step s; a
// lane instead takes the four consecutive k = 8 u + 4 (lane / 32) + j for steps
// 4 u + j (both operands agree on the order, and a sum does not care), which
// makes its operand reads 16 bytes wide.  Tiles are staged through registers
// into LDS rows of 32 + 4 floats.  K % 4 == 0 and N % 4 == 0.
// ---------------------------------------------------------------------------
// TM x TN: MFMA tiles per wavefront; the block tile is 64 TM x 64 TN.
template <int TM, int TN>
struct F32Cfg {
  static constexpr int BM = 64 * TM, BN = 64 * TN, BK = 32, THREADS = 256;
  static constexpr int LDK = BK + 4;               // floats per LDS row
  static constexpr int CPR = BK / 4;               // 16-byte chunks per row
  static constexpr int A_CHUNKS = BM * CPR / THREADS, B_CHUNKS = BN * CPR / THREADS;
  static constexpr size_t LDS_BYTES = 2ull * (BM + BN) * LDK * sizeof(float);
};

template <bool RELU, int TM, int TN>
__global__ __launch_bounds__(256) void grouped_gemm_f32_mfma_kernel(
    const float* __restrict__ A, const float* __restrict__ B,
    float* __restrict__ Cout, int R, int N, int K, int tiles_m, int tiles_n) {
  using Cfg = F32Cfg<TM, TN>;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, LDK = Cfg::LDK;
  constexpr int WTM = 32 * TM, WTN = 32 * TN;      // a wavefront's sub-tile
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* As = reinterpret_cast<float*>(smem_raw);  // [2][BM][LDK]
  float* Bs = As + 2 * BM * LDK;                   // [2][BN][LDK]
  const int tiles_per_e = tiles_m * tiles_n;
  const int e = blockIdx.x / tiles_per_e;
  const int rem = blockIdx.x - e * tiles_per_e;
  const int tn = rem / tiles_m, tm = rem - tn * tiles_m;
  const int row0 = tm * BM, col0 = tn * BN;
  const float* Ae = A + (int64_t)e * R * K;
  const float* Be = B + (int64_t)e * N * K;
  float* Ce = Cout + (int64_t)e * R * N;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  uint4 areg[Cfg::A_CHUNKS], breg[Cfg::B_CHUNKS];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < Cfg::A_CHUNKS; ++i) {
      const int c = tid + i * Cfg::THREADS;
      const int r = c / Cfg::CPR, gk = k0 + (c % Cfg::CPR) * 4;
      const int gr = min(row0 + r, R - 1);
      const uint4 v = *reinterpret_cast<const uint4*>(
          Ae + (int64_t)gr * K + min(gk, K - 4));
      areg[i] = gk < K ? v : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_CHUNKS; ++i) {
      const int c = tid + i * Cfg::THREADS;
      const int r = c / Cfg::CPR, gk = k0 + (c % Cfg::CPR) * 4;
      const int gr = min(col0 + r, N - 1);
      const uint4 v = *reinterpret_cast<const uint4*>(
          Be + (int64_t)gr * K + min(gk, K - 4));
      breg[i] = gk < K ? v : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < Cfg::A_CHUNKS; ++i) {
      const int c = tid + i * Cfg::THREADS;
      *reinterpret_cast<uint4*>(As + (buf * BM + c / Cfg::CPR) * LDK +
                                (c % Cfg::CPR) * 4) = areg[i];
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_CHUNKS; ++i) {
      const int c = tid + i * Cfg::THREADS;
      *reinterpret_cast<uint4*>(Bs + (buf * BN + c / Cfg::CPR) * LDK +
                                (c % Cfg::CPR) * 4) = breg[i];
    }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 4;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global((kt + 1) * BK);
    const float* as = As + (buf * BM + wm * WTM + frag_row) * LDK + frag_k;
    const float* bs = Bs + (buf * BN + wn * WTN + frag_row) * LDK + frag_k;
#pragma unroll
    for (int u = 0; u < BK / 8; ++u) {
      float4 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const float4*>(as + i * 32 * LDK + u * 8);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bfr[j] = *reinterpret_cast<const float4*>(bs + j * 32 * LDK + u * 8);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const float a = q == 0 ? af[i].x : q == 1 ? af[i].y
                            : q == 2 ? af[i].z : af[i].w;
            const float b = q == 0 ? bfr[j].x : q == 1 ? bfr[j].y
                            : q == 2 ? bfr[j].z : bfr[j].w;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, acc[i][j],
                                                             0, 0, 0);
          }
      }
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }
  const int m_l = lane & 31, n_l = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int grow = row0 + wm * WTM + i * 32 + m_l;
        const int gcol = col0 + wn * WTN + j * 32 + 8 * q + n_l;
        if (grow < R && gcol < N) {
          float4 v = make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1],
                                 acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
          if (RELU) {
            v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f);
            v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f);
          }
          *reinterpret_cast<float4*>(Ce + (int64_t)grow * N + gcol) = v;
        }
      }
}

// ---------------------------------------------------------------------------
// Plain FMA tile kernel (float32, and bf16 shapes the MFMA kernel rejects):
// 64 x 64 tile, 16-deep K step, each thread a 4 x 4 patch, float32 accumulate
// in k order.
// ---------------------------------------------------------------------------
template <typename T, bool RELU, typename TO = T>
__global__ __launch_bounds__(256) void grouped_gemm_simple_kernel(
    const T* __restrict__ A, const T* __restrict__ B, TO* __restrict__ Cout,
    int R, int N, int K, int tiles_m, int tiles_n) {
  __shared__ float As[16][64 + 4];
  __shared__ float Bs[16][64 + 4];
  const int tiles_per_e = tiles_m * tiles_n;
  const int e = blockIdx.x / tiles_per_e;
  const int rem = blockIdx.x - e * tiles_per_e;
  const int tn = rem / tiles_m, tm = rem - tn * tiles_m;
  const int row0 = tm * 64, col0 = tn * 64;
  const T* Ae = A + (int64_t)e * R * K;
  const T* Be = B + (int64_t)e * N * K;
  TO* Ce = Cout + (int64_t)e * R * N;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int c = tid + i * 256;
      int r = c >> 4, k = c & 15;
      int gr = row0 + r, gc = col0 + r, gk = k0 + k;
      As[k][r] = (gr < R && gk < K) ? load_f32<T>(Ae + (int64_t)gr * K + gk) : 0.f;
      Bs[k][r] = (gc < N && gk < K) ? load_f32<T>(Be + (int64_t)gc * K + gk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = row0 + ty * 4 + i;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int col = col0 + tx * 4 + j;
      if (row < R && col < N) {
        float v = round_to<TO>(acc[i][j]);
        if (RELU) v = v > 0.f ? v : 0.f;
        store_f32<TO>(Ce + (int64_t)row * N + col, v);
      }
    }
  }
}

// In-place activation on an already rounded tensor, for the activations that
// are not fused into the GEMM epilogue (everything except relu / linear).
template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(T* __restrict__ h,
                                                         int64_t n, int act) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride)
    store_f32<T>(h + i, apply_activation(load_f32<T>(h + i), act));
}

// out = act(pre), element by element (what activation_kernel does in place).
template <typename T>
__global__ __launch_bounds__(256) void activation_copy_kernel(
    const T* __restrict__ pre, T* __restrict__ out, int64_t n, int act) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride)
    store_f32<T>(out + i, apply_activation(load_f32<T>(pre + i), act));
}

// dh = dh * scale (when given), then dh = (h > 0) ? dh : 0 for ReLU experts --
// the hidden dropout and the ReLU of the forward pass seen from behind (h is
// the stored, already rounded activation: positive iff the pre-activation
// rounded to a positive value and the element was not dropped).
// (const_scale: one factor for every element that stays, in place of a scale
// tensor -- a dropout's noise where the ReLU mask already says which elements
// were kept.)
template <typename T>
__global__ __launch_bounds__(256) void hidden_grad_kernel(
    T* __restrict__ dh, const T* __restrict__ h, const T* __restrict__ scale,
    bool relu, int64_t n, float const_scale) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    if (relu && !(load_f32<T>(h + i) > 0.f)) {
      dh[i] = (T)0;
    } else if (scale) {
      store_f32<T>(dh + i, load_f32<T>(dh + i) * load_f32<T>(scale + i));
    } else if (const_scale != 1.0f) {
      store_f32<T>(dh + i, load_f32<T>(dh + i) * const_scale);
    }
  }
}

// h = h * factor (when given), then dropout: noise = (u < keep) ? inv_keep : 0,
// h = h * noise, each product rounded once to T.
template <typename T>
__global__ __launch_bounds__(256) void hidden_product_kernel(
    T* __restrict__ h, const T* __restrict__ factor,
    const T* __restrict__ uniform, float keep, float inv_keep,
    T* __restrict__ noise_out, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    float v = load_f32<T>(h + i);
    if (factor) {
      store_f32<T>(h + i, v * load_f32<T>(factor + i));
      v = load_f32<T>(h + i);
    }
    if (uniform) {
      const float noise = load_f32<T>(uniform + i) < keep ? inv_keep : 0.f;
      store_f32<T>(h + i, v * noise);
      if (noise_out) store_f32<T>(noise_out + i, noise);
    } 
  }
}

// d(act(v)) / dv in float32, from the pre-activation v.
__device__ __forceinline__ float activation_derivative(float v, int act) {
  switch (act) {
    case MESH_MOE_ACT_RELU:
      return v > 0.f ? 1.0f : 0.0f;
    case MESH_MOE_ACT_GELU: {
      const float k = 0.7978845608028654f;
      const float t = tanhf(k * (v + 0.044715f * v * v * v));
      const float du = k * (1.0f + 3.0f * 0.044715f * v * v);
      return 0.5f * (1.0f + t) + 0.5f * v * (1.0f - t * t) * du;
    }
    case MESH_MOE_ACT_SIGMOID: {
      const float sg = 1.0f / (1.0f + expf(-v));
      return sg * (1.0f - sg);
    }
    case MESH_MOE_ACT_TANH: {
      const float t = tanhf(v);
      return 1.0f - t * t;
    }
    case MESH_MOE_ACT_SWISH: {
      const float sg = 1.0f / (1.0f + expf(-v));
      return sg + v * sg * (1.0f - sg);
    }
    default:
      return 1.0f;
  }
}

// dpre = dh * factor * act'(pre), float32 arithmetic, one rounding.
template <typename T>
__global__ __launch_bounds__(256) void activation_backward_kernel(
    const T* __restrict__ dh, const T* __restrict__ pre,
    const T* __restrict__ factor, T* __restrict__ dpre, int64_t n, int act) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    float g = load_f32<T>(dh + i);
    if (factor) g *= load_f32<T>(factor + i);
    store_f32<T>(dpre + i, g * activation_derivative(load_f32<T>(pre + i), act));
  }
}

// The same for bf16 with 16-byte accesses: 8 elements per thread and step.
__global__ __launch_bounds__(256) void activation_backward_bf16x8_kernel(
    const uint4* __restrict__ dh, const uint4* __restrict__ pre,
    const uint4* __restrict__ factor, uint4* __restrict__ dpre, int64_t n8,
    int act) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += stride) {
    const uint4 g4 = load_streaming(dh + i), p4 = load_streaming(pre + i);
    uint4 f4 = make_uint4(0, 0, 0, 0);
    if (factor) f4 = load_streaming(factor + i);
    const uint32_t g[4] = {g4.x, g4.y, g4.z, g4.w}, p[4] = {p4.x, p4.y, p4.z, p4.w};
    const uint32_t f[4] = {f4.x, f4.y, f4.z, f4.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float g0 = __uint_as_float(g[j] << 16), g1 = __uint_as_float(g[j] & 0xffff0000u);
      if (factor) {
        g0 *= __uint_as_float(f[j] << 16);
        g1 *= __uint_as_float(f[j] & 0xffff0000u);
      }
      o[j] = f32x2_to_bf16x2(
          g0 * activation_derivative(__uint_as_float(p[j] << 16), act),
          g1 * activation_derivative(__uint_as_float(p[j] & 0xffff0000u), act));
    }
    store_streaming(dpre + i, make_uint4(o[0], o[1], o[2], o[3]));
  }
}

// hidden_grad_kernel, hidden_product_kernel and activation_kernel for bf16
// with 16-byte accesses (8 elements per thread and step; the same arithmetic
// and the same roundings element by element).
__global__ __launch_bounds__(256) void hidden_grad_bf16x8_kernel(
    uint4* __restrict__ dh, const uint4* __restrict__ h,
    const uint4* __restrict__ scale, bool relu, int64_t n8,
    float const_scale) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += stride) {
    float d[8], hv[8], sc[8];
    unpack16(load_streaming(dh + i), d, bf16_t());
    if (relu) unpack16(load_streaming(h + i), hv, bf16_t());
    if (scale) unpack16(load_streaming(scale + i), sc, bf16_t());
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (relu && !(hv[j] > 0.f)) d[j] = 0.f;
      else if (scale) d[j] = d[j] * sc[j];
      else d[j] = d[j] * const_scale;
    }
    store_streaming(dh + i, pack16(d, bf16_t()));
  }
}

__global__ __launch_bounds__(256) void hidden_product_bf16x8_kernel(
    uint4* __restrict__ h, const uint4* __restrict__ factor,
    const uint4* __restrict__ uniform, float keep, float inv_keep,
    uint4* __restrict__ noise_out, int64_t n8) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += stride) {
    float v[8], f[8], u[8], nz[8];
    unpack16(load_streaming(h + i), v, bf16_t());
    if (factor) {
      unpack16(load_streaming(factor + i), f, bf16_t());
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = round_to<bf16_t>(v[j] * f[j]);
    }
    if (uniform) {
      unpack16(load_streaming(uniform + i), u, bf16_t());
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        nz[j] = u[j] < keep ? inv_keep : 0.f;
        v[j] = v[j] * nz[j];
      }
      if (noise_out) store_streaming(noise_out + i, pack16(nz, bf16_t()));
    }
    store_streaming(h + i, pack16(v, bf16_t()));
  }
}

// (out may be the input: in place)
__global__ __launch_bounds__(256) void activation_bf16x8_kernel(
    const uint4* h, uint4* out, int64_t n8, int act) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += stride) {
    float v[8];
    unpack16(load_streaming(h + i), v, bf16_t());
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = apply_activation(v[j], act);
    store_streaming(out + i, pack16(v, bf16_t()));
  }
}

static bool x8_applies(int64_t n, int dtype, const void* a, const void* b,
                       const void* c, const void* d = nullptr) {
  return dtype == MESH_MOE_BF16 && n % 8 == 0 &&
         (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)d) & 15) == 0;
}
static int elementwise_blocks(int64_t n) {
  return (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
}

// dh = dh * scale, then the ReLU mask of h (hidden_grad_kernel's contract)
static int launch_hidden_grad(void* dh, const void* h, const void* scale,
                              bool relu, int64_t n, int dtype, hipStream_t st,
                              float const_scale = 1.0f) {
  if (x8_applies(n, dtype, dh, h, scale))
    hidden_grad_bf16x8_kernel<<<elementwise_blocks(n / 8), 256, 0, st>>>(
        (uint4*)dh, (const uint4*)h, (const uint4*)scale, relu, n / 8,
        const_scale);
  else if (dtype == MESH_MOE_F32)
    hidden_grad_kernel<float><<<elementwise_blocks(n), 256, 0, st>>>(
        (float*)dh, (const float*)h, (const float*)scale, relu, n, const_scale);
  else
    hidden_grad_kernel<bf16_t><<<elementwise_blocks(n), 256, 0, st>>>(
        (bf16_t*)dh, (const bf16_t*)h, (const bf16_t*)scale, relu, n,
        const_scale);
  MOE_CHECK_LAUNCH("hidden gradient (mask / scale)");
  return 0;
}

// h = act(h) in place
static int launch_activation(void* h, int64_t n, int act, int dtype,
                             hipStream_t st) {
  if (x8_applies(n, dtype, h, nullptr, nullptr))
    activation_bf16x8_kernel<<<elementwise_blocks(n / 8), 256, 0, st>>>(
        (const uint4*)h, (uint4*)h, n / 8, act);
  else if (dtype == MESH_MOE_F32)
    activation_kernel<float><<<elementwise_blocks(n), 256, 0, st>>>((float*)h, n,
                                                                    act);
  else
    activation_kernel<bf16_t><<<elementwise_blocks(n), 256, 0, st>>>((bf16_t*)h,
                                                                     n, act);
  MOE_CHECK_LAUNCH("activation");
  return 0;
}

template <int BM, int BN, int BK>
static int launch_mfma(const bf16_t* A, const bf16_t* B, bf16_t* C, int E,
                       int R, int N, int K, bool relu, hipStream_t st) {
  using Cfg = GemmCfg<BM, BN, BK>;
  const int tiles_m = (R + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn: too many tiles (%lld)", (long long)blocks);
  if (relu) {
    auto k = grouped_gemm_bf16_kernel<BM, BN, BK, true>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, 256, Cfg::LDS_BYTES, st>>>(A, B, C, R, N, K, tiles_m,
                                                      tiles_n);
  } else {
    auto k = grouped_gemm_bf16_kernel<BM, BN, BK, false>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, 256, Cfg::LDS_BYTES, st>>>(A, B, C, R, N, K, tiles_m,
                                                      tiles_n);
  }
  MOE_CHECK_LAUNCH("expert_ffn (mfma)");
  return 0;
}

template <int BM, int BN, int WN, int WM = 2>
static int launch_dma(const bf16_t* A, const bf16_t* B, bf16_t* C, int E,
                      int R, int N, int K, bool relu, hipStream_t st) {
  using Cfg = DmaCfg<BM, BN, WN, WM>;
  const int tiles_m = (R + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn: too many tiles (%lld)", (long long)blocks);
  if (relu) {
    auto k = grouped_gemm_bf16_dma_kernel<BM, BN, WN, true, WM>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(A, B, C, R, N, K, tiles_m,
                                                      tiles_n);
  } else {
    auto k = grouped_gemm_bf16_dma_kernel<BM, BN, WN, false, WM>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(A, B, C, R, N, K, tiles_m,
                                                      tiles_n);
  }
  MOE_CHECK_LAUNCH("expert_ffn (mfma, direct-to-LDS)");
  return 0;
}

// Compute units of the current device (one persistent block per CU: a block
// takes all of a CU's LDS); 0 on failure.
static int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess || n < 1) {
      set_error("expert_ffn: cannot query the number of compute units");
      return 0;
    }
    cus = n;
  }
  return cus;
}

// C[e] [R, N] = A[e]^T . B[e] with A[e] [K, R] and B[e] [K, N] (both with the
// reduction index outermost); true if the K-major ring kernel takes the shape.
static bool kmajor_path_applies(const void* A, const void* B, const void* C,
                                int R, int N, int K, int dtype) {
  return dtype == MESH_MOE_BF16 && K >= 1 &&
         R % 8 == 0 && N % 8 == 0 && R >= 128 && N >= 128 &&
         (int64_t)R * K < (1LL << 31) && (int64_t)N * K < (1LL << 31) &&
         (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0;
}

static int launch_ring_kmajor(const bf16_t* A, const bf16_t* B, bf16_t* C,
                              int E, int R, int N, int K, hipStream_t st,
                              const int32_t* k_extent = nullptr) {
  using Cfg = RingCfg;
  const int tiles_m = (R + Cfg::BM - 1) / Cfg::BM;
  const int tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  const int64_t tiles = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(tiles <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn_backward: too many tiles (%lld)", (long long)tiles);
  const int cus = compute_units();
  if (cus == 0) return MESH_MOE_E_HIP;
  const unsigned blocks = (unsigned)(tiles < cus ? tiles : cus);
  auto k = grouped_gemm_bf16_ring_kernel<false, false, true>;
  MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
  k<<<blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(
      A, B, C, R, N, K, tiles_m, tiles_n, (int)tiles, nullptr, nullptr,
      nullptr, nullptr, k_extent, 1.0f);
  MOE_CHECK_LAUNCH("expert_ffn_backward (mfma, K-major operands)");
  return 0;
}

static int launch_ring(const bf16_t* A, const bf16_t* B, bf16_t* C, int E,
                       int R, int N, int K, bool relu, hipStream_t st,
                       const int32_t* row_map = nullptr,
                       const bf16_t* zero_row = nullptr,
                       const bf16_t* mask_src = nullptr,
                       const int32_t* tile_list = nullptr,
                       float mask_scale = 1.0f) {
  using Cfg = RingCfg;
  const int tiles_m = (R + Cfg::BM - 1) / Cfg::BM;
  const int tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  const int64_t tiles = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(tiles <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn: too many tiles (%lld)", (long long)tiles);
  const int cus = compute_units();
  if (cus == 0) return MESH_MOE_E_HIP;
  const unsigned blocks = (unsigned)(tiles < cus ? tiles : cus);
  if (tile_list != nullptr && mask_src != nullptr) {
    MOE_REQUIRE(!relu && row_map == nullptr, MESH_MOE_E_ARG,
                "expert_ffn: masked result with relu or gathered rows");
    auto k = grouped_gemm_bf16_ring_kernel<false, false, false, true, true>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n, (int)tiles, nullptr, nullptr,
        mask_src, tile_list, nullptr, mask_scale);
    MOE_CHECK_LAUNCH("expert_ffn (mfma, listed tiles, masked result)");
    return 0;
  }
  if (tile_list != nullptr) {
    // listed tiles: the first GEMM gathers its rows, the second does not
#define MOE_RING_LISTED(RELU_, GATHER_)                                        \
  do {                                                                         \
    auto k = grouped_gemm_bf16_ring_kernel<RELU_, GATHER_, false, false, true>; \
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);                                          \
    k<<<blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(                           \
        A, B, C, R, N, K, tiles_m, tiles_n, (int)tiles, row_map, zero_row,     \
        nullptr, tile_list, nullptr, 1.0f);                                    \
  } while (0)
    if (row_map != nullptr) {
      if (relu) MOE_RING_LISTED(true, true);
      else MOE_RING_LISTED(false, true);
    } else {
      if (relu) MOE_RING_LISTED(true, false);
      else MOE_RING_LISTED(false, false);
    }
#undef MOE_RING_LISTED
    MOE_CHECK_LAUNCH("expert_ffn (mfma, listed tiles)");
    return 0;
  }
  if (mask_src != nullptr) {
    MOE_REQUIRE(!relu && row_map == nullptr, MESH_MOE_E_ARG,
                "expert_ffn: masked result with relu or gathered rows");
    auto k = grouped_gemm_bf16_ring_kernel<false, false, false, true>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n, (int)tiles, nullptr, nullptr,
        mask_src, nullptr, nullptr, mask_scale);
    MOE_CHECK_LAUNCH("expert_ffn (mfma, masked result)");
    return 0;
  }
  // an expert's last row tile is partly empty: the instantiation that skips
  // its empty 32-row pieces
  const bool tails = R % Cfg::BM != 0;
#define MOE_RING_PLAIN(RELU_, GATHER_, TAILS_)                                 \
  do {                                                                         \
    auto k = grouped_gemm_bf16_ring_kernel<RELU_, GATHER_, false, false,       \
                                           false, TAILS_>;                     \
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);                                          \
    k<<<blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(                           \
        A, B, C, R, N, K, tiles_m, tiles_n, (int)tiles, row_map, zero_row,     \
        nullptr, nullptr, nullptr, 1.0f);                                      \
  } while (0)
#define MOE_RING_PLAIN_T(RELU_, GATHER_)                                       \
  do {                                                                         \
    if (tails) MOE_RING_PLAIN(RELU_, GATHER_, true);                           \
    else MOE_RING_PLAIN(RELU_, GATHER_, false);                                \
  } while (0)
  if (row_map != nullptr) {
    if (relu) MOE_RING_PLAIN_T(true, true);
    else MOE_RING_PLAIN_T(false, true);
    MOE_CHECK_LAUNCH("expert_ffn (mfma, gathered rows)");
    return 0;
  }
  if (relu) MOE_RING_PLAIN_T(true, false);
  else MOE_RING_PLAIN_T(false, false);
#undef MOE_RING_PLAIN_T
#undef MOE_RING_PLAIN
  MOE_CHECK_LAUNCH("expert_ffn (mfma, spread direct-to-LDS loads)");
  return 0;
}

template <int TM, int TN>
static int launch_f32_mfma_tile(const float* A, const float* B, float* C, int E,
                                int R, int N, int K, bool relu, hipStream_t st) {
  using Cfg = F32Cfg<TM, TN>;
  const int tiles_m = (R + Cfg::BM - 1) / Cfg::BM;
  const int tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn: too many tiles (%lld)", (long long)blocks);
  if (relu) {
    auto k = grouped_gemm_f32_mfma_kernel<true, TM, TN>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n);
  } else {
    auto k = grouped_gemm_f32_mfma_kernel<false, TM, TN>;
    MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
    k<<<(unsigned)blocks, Cfg::THREADS, Cfg::LDS_BYTES, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n);
  }
  MOE_CHECK_LAUNCH("expert_ffn (float32 mfma)");
  return 0;
}

// Block tile of the float32 kernel: 128 x 128, 64 x 128 or 64 x 64.  The
// kernel is bound by the float32 matrix pipes (a 32 x 32 x 2 MFMA takes 64
// cycles), so its time is rounds of tiles over the compute units times the
// tile's area; small launches want small tiles (less padding of the row count,
// fewer idle compute units in the last round).
static int launch_f32_mfma(const float* A, const float* B, float* C, int E,
                           int R, int N, int K, bool relu, hipStream_t st) {
  const int cus = compute_units();
  if (cus == 0) return MESH_MOE_E_HIP;
  static const int shapes[3][2] = {{2, 2}, {1, 2}, {1, 1}};
  int best = 0;
  double best_cost = 0;
  int64_t best_tiles = 0;
  for (int i = 0; i < 3; ++i) {
    const int bm = 64 * shapes[i][0], bn = 64 * shapes[i][1];
    const int64_t tiles = (int64_t)E * ((R + bm - 1) / bm) * ((N + bn - 1) / bn);
    const double cost = (double)((tiles + cus - 1) / cus) * bm * bn;
    // a smaller tile when it saves time by this count, or costs the same while
    // the larger one leaves compute units with fewer than two blocks to
    // overlap (measured at 8 experts x 320 rows, 2048 x 512: 64 x 64 tiles
    // 0.149 ms for both launches, 64 x 128 0.157, 128 x 128 0.228)
    if (i == 0 || cost < 0.95 * best_cost ||
        (cost <= best_cost && best_tiles < 2 * (int64_t)cus)) {
      best = i;
      best_cost = cost;
      best_tiles = tiles;
    }
  }
  switch (best) {
    case 0: return launch_f32_mfma_tile<2, 2>(A, B, C, E, R, N, K, relu, st);
    case 1: return launch_f32_mfma_tile<1, 2>(A, B, C, E, R, N, K, relu, st);
    default: return launch_f32_mfma_tile<1, 1>(A, B, C, E, R, N, K, relu, st);
  }
}

template <typename T>
static int launch_simple(const T* A, const T* B, T* C, int E, int R, int N,
                         int K, bool relu, hipStream_t st) {
  const int tiles_m = (R + 63) / 64, tiles_n = (N + 63) / 64;
  const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn: too many tiles (%lld)", (long long)blocks);
  if (relu)
    grouped_gemm_simple_kernel<T, true><<<(unsigned)blocks, 256, 0, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n);
  else
    grouped_gemm_simple_kernel<T, false><<<(unsigned)blocks, 256, 0, st>>>(
        A, B, C, R, N, K, tiles_m, tiles_n);
  MOE_CHECK_LAUNCH("expert_ffn (fma)");
  return 0;
}

// C[e] = act(A[e] . B[e]^T) for every expert.
// relu_mask_src (same shape and dtype as C): the kernels that can zero the
// elements of C whose mask_src element is not positive while they write C do so
// and set *mask_applied; otherwise the caller runs the mask as a pass of its own.
static int grouped_gemm(const void* A, const void* B, void* C, int E, int R,
                        int N, int K, int act, int dtype, hipStream_t st,
                        const void* relu_mask_src = nullptr,
                        bool* mask_applied = nullptr, float mask_scale = 1.0f) {
  const bool relu = act == MESH_MOE_ACT_RELU;
  int rc;
  if (mask_applied) *mask_applied = false;
  if (dtype == MESH_MOE_F32) {
    if (K % 4 == 0 && N % 4 == 0 && K >= 32 && R >= 32 && N >= 32 &&
        (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) % 16 == 0))
      rc = launch_f32_mfma((const float*)A, (const float*)B, (float*)C, E, R,
                           N, K, relu, st);
    else
      rc = launch_simple<float>((const float*)A, (const float*)B, (float*)C, E,
                                R, N, K, relu, st);
  } else {
    const bool mfma_ok =
        (K % 8 == 0) && (N % 8 == 0) &&
        (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) % 16 == 0);
    if (!mfma_ok)
      rc = launch_simple<bf16_t>((const bf16_t*)A, (const bf16_t*)B,
                                 (bf16_t*)C, E, R, N, K, relu, st);
    else if (N >= 256 && R >= 128 && K % 64 == 0 &&
             (int64_t)R * K < (1LL << 31) && (int64_t)N * K < (1LL << 31)) {
      // direct-to-LDS kernels; the persistent 256-row kernel unless 128-row
      // tiles save more than a fifth of the padded rows (at 640 rows per
      // expert, 3 x 256 against 5 x 128, the persistent kernel still wins:
      // 0.43 against 0.50 ms for both GEMMs of benchmark config 2)
      const bf16_t *a = (const bf16_t*)A, *b = (const bf16_t*)B;
      bf16_t* c = (bf16_t*)C;
      const int pad256 = (R + 255) / 256 * 256, pad128 = (R + 127) / 128 * 128;
      // 256 x 256 tiles run 8 wavefronts (two per SIMD, 128 x 64 sub-tiles)
      // with the loads spread over the MFMA steps
      if (pad128 * 5 < pad256 * 4) {
        rc = launch_dma<128, 256, 2>(a, b, c, E, R, N, K, relu, st);
      } else if (relu_mask_src != nullptr && mask_applied != nullptr && !relu &&
                 ((uintptr_t)relu_mask_src % 16) == 0) {
        rc = launch_ring(a, b, c, E, R, N, K, false, st, nullptr, nullptr,
                         (const bf16_t*)relu_mask_src, nullptr, mask_scale);
        *mask_applied = rc == 0;
      } else {
        rc = launch_ring(a, b, c, E, R, N, K, relu, st);
      }
    } else if (R >= 1024 && N >= 1024)
      rc = launch_mfma<256, 256, 64>((const bf16_t*)A, (const bf16_t*)B,
                                     (bf16_t*)C, E, R, N, K, relu, st);
    else
      rc = launch_mfma<128, 128, 64>((const bf16_t*)A, (const bf16_t*)B,
                                     (bf16_t*)C, E, R, N, K, relu, st);
  }
  if (rc != 0) return rc;
  if (act != MESH_MOE_ACT_RELU && act != MESH_MOE_ACT_LINEAR)
    return launch_activation(C, (int64_t)E * R * N, act, dtype, st);
  return 0;
}

// Batched C[e] = A[e] . B[e]^T for the other source files (attention): `dtype`
// operands, `dtype` result or, with out_f32, a float32 result.
int batched_gemm_nt(const void* A, const void* B, void* C, int E, int R, int N,
                    int K, int dtype, bool out_f32, hipStream_t st) {
  if (dtype == MESH_MOE_F32 || !out_f32)
    return grouped_gemm(A, B, C, E, R, N, K, MESH_MOE_ACT_LINEAR, dtype, st);
  if (!(K % 8 == 0 && N % 8 == 0 &&
        (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) % 16 == 0))) {
    // shapes the matrix-core kernel does not take (e.g. a key / value size
    // that is not a multiple of 8): the plain tile kernel, bf16 in, float32 out
    const int tiles_m = (R + 63) / 64, tiles_n = (N + 63) / 64;
    const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
    MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
                "batched_gemm_nt: too many tiles (%lld)", (long long)blocks);
    grouped_gemm_simple_kernel<bf16_t, false, float>
        <<<(unsigned)blocks, 256, 0, st>>>((const bf16_t*)A, (const bf16_t*)B,
                                           (float*)C, R, N, K, tiles_m, tiles_n);
    MOE_CHECK_LAUNCH("batched_gemm_nt (fma, float32 result)");
    return 0;
  }
  using Cfg = GemmCfg<128, 128, 64>;
  const int tiles_m = (R + 127) / 128, tiles_n = (N + 127) / 128;
  const int64_t blocks = (int64_t)tiles_m * tiles_n * E;
  MOE_REQUIRE(blocks <= 0x7fffffffLL, MESH_MOE_E_UNSUPPORTED,
              "batched_gemm_nt: too many tiles (%lld)", (long long)blocks);
  auto k = grouped_gemm_bf16_kernel<128, 128, 64, false, true>;
  MOE_ALLOW_LDS(k, Cfg::LDS_BYTES);
  k<<<(unsigned)blocks, 256, Cfg::LDS_BYTES, st>>>(
      (const bf16_t*)A, (const bf16_t*)B, C, R, N, K, tiles_m, tiles_n);
  MOE_CHECK_LAUNCH("batched_gemm_nt (mfma, float32 result)");
  return 0;
}

}  // namespace mesh_moe

using namespace mesh_moe;

extern "C" int mesh_moe_expert_ffn(const void* expert_in, const void* wi_packed,
                                   const void* wo_packed, void* h, void* y,
                                   int E, int R, int M, int H, int N,
                                   int activation, int dtype, void* stream) {
  MOE_REQUIRE(expert_in && wi_packed && wo_packed && h && y, MESH_MOE_E_ARG,
              "expert_ffn: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "expert_ffn: bad dtype %d",
              dtype);
  MOE_REQUIRE(E >= 1 && R >= 1 && M >= 1 && H >= 1 && N >= 1, MESH_MOE_E_ARG,
              "expert_ffn: bad sizes E=%d R=%d M=%d H=%d N=%d", E, R, M, H, N);
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "expert_ffn: unknown activation %d", activation);
  hipStream_t st = (hipStream_t)stream;
  int rc = grouped_gemm(expert_in, wi_packed, h, E, R, H, M, activation, dtype,
                        st);
  if (rc != 0) return rc;
  return grouped_gemm(h, wo_packed, y, E, R, N, H, MESH_MOE_ACT_LINEAR, dtype,
                      st);
}

namespace mesh_moe {

// ---------------------------------------------------------------------------
// Dispatch folded into the first expert GEMM: slot -> token map.
// ---------------------------------------------------------------------------
__global__ void slot_map_clear_kernel(int32_t* map, int64_t n, bf16_t* zero_row,
                                      int m) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = i0; i < n; i += stride) map[i] = -1;
  for (int64_t i = i0; i < m; i += stride) zero_row[i] = 0;
}

// one thread per (token, choice): a kept choice whose activation-dtype gate is
// not 0 owns slot [idx][g][pos] (transformer/moe.py:1510-1511: the dispatch
// tensor is the combine tensor cast to bool)
__global__ void slot_map_kernel(const int32_t* __restrict__ idx,
                                const int32_t* __restrict__ pos,
                                const float* __restrict__ gate,
                                const uint8_t* __restrict__ kept,
                                int32_t* __restrict__ map, int64_t tokens,
                                int S, int C, int64_t rows_per_expert) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= tokens * 2) return;
  if (!kept[i] || round_to<bf16_t>(gate[i]) == 0.0f) return;
  const int64_t t = i >> 1;
  const int64_t g = t / S;
  map[(int64_t)idx[i] * rows_per_expert + g * C + pos[i]] = (int32_t)t;
}

// ---------------------------------------------------------------------------
// Compacted rows: expert e's occupied slots, groups in order, slots in order,
// become rows 0 .. rows_used[e] - 1 of its row range.
// row_offsets[e][g] = sum over g' < g of fill[g'][e]; one block per expert.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void row_offsets_kernel(
    const int32_t* __restrict__ fill, int32_t* __restrict__ row_offsets,
    int32_t* __restrict__ rows_used, int G, int E) {
  __shared__ int32_t part[256];
  const int e = blockIdx.x, tid = threadIdx.x;
  const int per = (G + 255) / 256;
  const int g0 = min(G, tid * per), g1 = min(G, g0 + per);
  int sum = 0;
  for (int g = g0; g < g1; ++g) sum += fill[(int64_t)g * E + e];
  part[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int i = 0; i < 256; ++i) {
      const int v = part[i];
      part[i] = run;
      run += v;
    }
    rows_used[e] = run;
  }
  __syncthreads();
  int run = part[tid];
  for (int g = g0; g < g1; ++g) {
    row_offsets[(int64_t)e * G + g] = run;
    run += fill[(int64_t)g * E + e];
  }
}

// One thread per (token, choice), as slot_map_kernel, onto the compacted rows.
__global__ void slot_map_compact_kernel(const int32_t* __restrict__ idx,
                                        const int32_t* __restrict__ pos,
                                        const float* __restrict__ gate,
                                        const uint8_t* __restrict__ kept,
                                        const int32_t* __restrict__ row_offsets,
                                        int32_t* __restrict__ map,
                                        int64_t tokens, int S, int G,
                                        int64_t rows_per_expert) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= tokens * 2) return;
  if (!kept[i] || round_to<bf16_t>(gate[i]) == 0.0f) return;
  const int64_t t = i >> 1;
  const int64_t g = t / S;
  const int e = idx[i];
  map[(int64_t)e * rows_per_expert + row_offsets[(int64_t)e * G + g] + pos[i]] =
      (int32_t)t;
}

// The tiles that hold occupied rows, in the order of the full tile numbering
// ((expert, N tile, M tile), M tile fastest): list[-1] = their number.  One
// block; E <= 1024.
__global__ __launch_bounds__(1024) void tile_list_kernel(
    const int32_t* __restrict__ rows_used, int32_t* __restrict__ list, int E,
    int tiles_m, int tiles_n, int bm) {
  __shared__ int32_t mt[1024], pre[1025];
  const int tid = threadIdx.x;
  if (tid < E) mt[tid] = min(tiles_m, (rows_used[tid] + bm - 1) / bm);
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { pre[e] = run; run += mt[e]; }
    pre[E] = run;
    list[-1] = run * tiles_n;
  }
  __syncthreads();
  const int total = E * tiles_n * tiles_m;
  for (int i = tid; i < total; i += blockDim.x) {
    const int tm = i % tiles_m, rest = i / tiles_m;
    const int tn = rest % tiles_n, e = rest / tiles_n;
    if (tm < mt[e]) list[tiles_n * pre[e] + tn * mt[e] + tm] = i;
  }
}

// rows_used[e] from the row offsets of the last group and its fill count
__global__ void rows_used_kernel(const int32_t* __restrict__ fill,
                                 const int32_t* __restrict__ row_offsets,
                                 int32_t* __restrict__ rows_used, int G, int E) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < E)
    rows_used[e] = row_offsets[(int64_t)e * G + G - 1] +
                   fill[(int64_t)(G - 1) * E + e];
}

static bool ring_path_applies(int R, int N, int K) {
  const int pad256 = (R + 255) / 256 * 256, pad128 = (R + 127) / 128 * 128;
  return N >= 256 && R >= 128 && K % 64 == 0 && K % 8 == 0 && N % 8 == 0 &&
         pad128 * 5 >= pad256 * 4 && (int64_t)N * K < (1LL << 31);
}

}  // namespace mesh_moe

extern "C" size_t mesh_moe_dispatched_expert_ffn_workspace_bytes(int G, int E,
                                                                 int C, int M) {
  if (G < 1 || E < 1 || C < 1 || M < 1) return 0;
  return sizeof(int32_t) * (size_t)E * G * C + sizeof(bf16_t) * (size_t)M + 512;
}

extern "C" int mesh_moe_dispatched_expert_ffn(
    const void* x, const int32_t* idx, const int32_t* pos, const float* gate,
    const uint8_t* kept, const void* wi_packed, const void* wo_packed, void* h,
    void* y, void* workspace, size_t workspace_bytes, int G, int S, int E, int C,
    int M, int H, int N, int activation, int dtype, void* stream) {
  MOE_REQUIRE(x && idx && pos && gate && kept && wi_packed && wo_packed && h &&
                  y && workspace, MESH_MOE_E_ARG,
              "dispatched_expert_ffn: null pointer");
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1 && H >= 1 && N >= 1,
              MESH_MOE_E_ARG, "dispatched_expert_ffn: bad sizes");
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "dispatched_expert_ffn: unknown activation %d",
              activation);
  const int64_t rows = (int64_t)G * C;
  MOE_REQUIRE(dtype == MESH_MOE_BF16 && rows <= 0x7fffffffLL &&
                  (int64_t)G * S <= 0x7fffffffLL &&
                  ring_path_applies((int)rows, H, M) &&
                  (((uintptr_t)x | (uintptr_t)wi_packed | (uintptr_t)h) % 16 == 0),
              MESH_MOE_E_UNSUPPORTED,
              "dispatched_expert_ffn: needs bf16 and a first GEMM the 256 x 256 "
              "direct-to-LDS kernel takes (rows=%lld M=%d H=%d)",
              (long long)rows, M, H);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_dispatched_expert_ffn_workspace_bytes(G, E, C, M),
              MESH_MOE_E_ARG, "dispatched_expert_ffn: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  const int R = (int)rows;
  int32_t* map = (int32_t*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  bf16_t* zero_row =
      (bf16_t*)(((uintptr_t)(map + (size_t)E * R) + 255) & ~(uintptr_t)255);
  const int64_t n_map = (int64_t)E * R;
  const unsigned cb = (unsigned)((n_map + 255) / 256 < 4096 ? (n_map + 255) / 256
                                                            : 4096);
  slot_map_clear_kernel<<<cb, 256, 0, st>>>(map, n_map, zero_row, M);
  MOE_CHECK_LAUNCH("dispatched_expert_ffn (clear)");
  const int64_t pairs = (int64_t)G * S * 2;
  slot_map_kernel<<<(unsigned)((pairs + 255) / 256), 256, 0, st>>>(
      idx, pos, gate, kept, map, (int64_t)G * S, S, C, rows);
  MOE_CHECK_LAUNCH("dispatched_expert_ffn (slot map)");
  const bool relu = activation == MESH_MOE_ACT_RELU;
  int rc = launch_ring((const bf16_t*)x, (const bf16_t*)wi_packed, (bf16_t*)h,
                       E, R, H, M, relu, st, map, zero_row);
  if (rc != 0) return rc;
  if (!relu && activation != MESH_MOE_ACT_LINEAR) {
    rc = launch_activation(h, (int64_t)E * R * H, activation, dtype, st);
    if (rc != 0) return rc;
  }
  return grouped_gemm(h, wo_packed, y, E, R, N, H, MESH_MOE_ACT_LINEAR, dtype,
                      st);
}

static size_t compact_ffn_tiles(int E, int R, int H, int N) {
  const size_t tm = (size_t)(R + RingCfg::BM - 1) / RingCfg::BM;
  return (size_t)E * tm * ((size_t)(H + RingCfg::BN - 1) / RingCfg::BN +
                           (size_t)(N + RingCfg::BN - 1) / RingCfg::BN);
}

extern "C" size_t mesh_moe_compact_expert_ffn_workspace_bytes(int G, int E,
                                                              int C, int M,
                                                              int H, int N) {
  if (G < 1 || E < 1 || C < 1 || M < 1 || H < 1 || N < 1) return 0;
  const int64_t rows = (int64_t)G * C;
  if (rows > 0x7fffffffLL) return 0;
  return sizeof(int32_t) * ((size_t)E * rows + (size_t)E +
                            compact_ffn_tiles(E, (int)rows, H, N) + 2 * 64) +
         sizeof(bf16_t) * (size_t)M + 6 * 256;
}

extern "C" int mesh_moe_compact_expert_ffn(
    const void* x, const int32_t* idx, const int32_t* pos, const float* gate,
    const uint8_t* kept, const int32_t* fill, const void* wi_packed,
    const void* wo_packed, void* h, void* y, int32_t* row_offsets,
    const void* hidden_uniform, float keep_prob, void* noise_out,
    void* workspace, size_t workspace_bytes, int G, int S, int E, int C, int M,
    int H, int N, int activation, int dtype, void* stream) {
  MOE_REQUIRE(x && idx && pos && gate && kept && fill && wi_packed &&
                  wo_packed && h && y && row_offsets && workspace,
              MESH_MOE_E_ARG, "compact_expert_ffn: null pointer");
  MOE_REQUIRE(!noise_out || hidden_uniform, MESH_MOE_E_ARG,
              "compact_expert_ffn: noise_out without hidden_uniform");
  MOE_REQUIRE(!hidden_uniform || (keep_prob > 0.f && keep_prob <= 1.f),
              MESH_MOE_E_ARG, "compact_expert_ffn: keep_prob %g outside (0, 1]",
              (double)keep_prob);
  MOE_REQUIRE(G >= 1 && S >= 1 && E >= 1 && C >= 1 && M >= 1 && H >= 1 && N >= 1,
              MESH_MOE_E_ARG, "compact_expert_ffn: bad sizes");
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "compact_expert_ffn: unknown activation %d",
              activation);
  const int64_t rows = (int64_t)G * C;
  MOE_REQUIRE(dtype == MESH_MOE_BF16 && rows <= 0x7fffffffLL && E <= 1024 &&
                  (int64_t)G * S <= 0x7fffffffLL &&
                  ring_path_applies((int)rows, H, M) &&
                  ring_path_applies((int)rows, N, H) &&
                  (((uintptr_t)x | (uintptr_t)wi_packed | (uintptr_t)wo_packed |
                    (uintptr_t)h | (uintptr_t)y) % 16 == 0),
              MESH_MOE_E_UNSUPPORTED,
              "compact_expert_ffn: needs bf16, at most 1024 experts and GEMMs "
              "the 256 x 256 direct-to-LDS kernel takes (rows=%lld M=%d H=%d "
              "N=%d)", (long long)rows, M, H, N);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_compact_expert_ffn_workspace_bytes(
                                     G, E, C, M, H, N),
              MESH_MOE_E_ARG, "compact_expert_ffn: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  const int R = (int)rows;
  auto up = [](uintptr_t q) { return (q + 255) & ~(uintptr_t)255; };
  int32_t* map = (int32_t*)up((uintptr_t)workspace);
  int32_t* rows_used = (int32_t*)up((uintptr_t)(map + (size_t)E * R));
  const int tiles_m = (R + RingCfg::BM - 1) / RingCfg::BM;
  const int tn1 = (H + RingCfg::BN - 1) / RingCfg::BN;
  const int tn2 = (N + RingCfg::BN - 1) / RingCfg::BN;
  // each list is preceded by its length (and padding up to 256 bytes)
  int32_t* list1 = (int32_t*)up((uintptr_t)(rows_used + E)) + 64;
  int32_t* list2 = (int32_t*)up((uintptr_t)(list1 + (size_t)E * tiles_m * tn1)) + 64;
  bf16_t* zero_row = (bf16_t*)up((uintptr_t)(list2 + (size_t)E * tiles_m * tn2));
  row_offsets_kernel<<<E, 256, 0, st>>>(fill, row_offsets, rows_used, G, E);
  MOE_CHECK_LAUNCH("compact_expert_ffn (row offsets)");
  const int64_t n_map = (int64_t)E * R;
  const unsigned cb = (unsigned)((n_map + 255) / 256 < 4096 ? (n_map + 255) / 256
                                                            : 4096);
  slot_map_clear_kernel<<<cb, 256, 0, st>>>(map, n_map, zero_row, M);
  MOE_CHECK_LAUNCH("compact_expert_ffn (clear)");
  const int64_t pairs = (int64_t)G * S * 2;
  slot_map_compact_kernel<<<(unsigned)((pairs + 255) / 256), 256, 0, st>>>(
      idx, pos, gate, kept, row_offsets, map, (int64_t)G * S, S, G, rows);
  MOE_CHECK_LAUNCH("compact_expert_ffn (slot map)");
  tile_list_kernel<<<1, 1024, 0, st>>>(rows_used, list1, E, tiles_m, tn1,
                                       RingCfg::BM);
  MOE_CHECK_LAUNCH("compact_expert_ffn (tile list 1)");
  tile_list_kernel<<<1, 1024, 0, st>>>(rows_used, list2, E, tiles_m, tn2,
                                       RingCfg::BM);
  MOE_CHECK_LAUNCH("compact_expert_ffn (tile list 2)");
  const bool relu = activation == MESH_MOE_ACT_RELU;
  int rc = launch_ring((const bf16_t*)x, (const bf16_t*)wi_packed, (bf16_t*)h,
                       E, R, H, M, relu, st, map, zero_row, nullptr, list1);
  if (rc != 0) return rc;
  if (!relu && activation != MESH_MOE_ACT_LINEAR) {
    // (the pass also runs over the rows no listed tile wrote: they hold
    // unspecified values before and after, and nothing reads them)
    rc = launch_activation(h, (int64_t)E * R * H, activation, dtype, st);
    if (rc != 0) return rc;
  }
  if (hidden_uniform != nullptr) {
    // the hidden dropout, element for element of the [E, G*C, H] buffer (the
    // noise of a slot is the one drawn at its compacted row)
    rc = mesh_moe_hidden_product(h, nullptr, hidden_uniform, keep_prob,
                                 noise_out, (int64_t)E * R * H, dtype, stream);
    if (rc != 0) return rc;
  }
  return launch_ring((const bf16_t*)h, (const bf16_t*)wo_packed, (bf16_t*)y, E,
                     R, N, H, false, st, nullptr, nullptr, nullptr, list2);
}

extern "C" int mesh_moe_expert_linear(const void* a, const void* w_packed,
                                      void* y, int E, int R, int K, int N,
                                      int activation, int dtype, void* stream) {
  MOE_REQUIRE(a && w_packed && y, MESH_MOE_E_ARG, "expert_linear: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "expert_linear: bad dtype %d",
              dtype);
  MOE_REQUIRE(E >= 1 && R >= 1 && K >= 1 && N >= 1, MESH_MOE_E_ARG,
              "expert_linear: bad sizes E=%d R=%d K=%d N=%d", E, R, K, N);
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "expert_linear: unknown activation %d",
              activation);
  return grouped_gemm(a, w_packed, y, E, R, N, K, activation, dtype,
                      (hipStream_t)stream);
}

extern "C" int mesh_moe_hidden_product(void* h, const void* factor,
                                       const void* uniform, float keep_prob,
                                       void* noise_out, int64_t n, int dtype,
                                       void* stream) {
  MOE_REQUIRE(h, MESH_MOE_E_ARG, "hidden_product: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "hidden_product: bad dtype %d", dtype);
  MOE_REQUIRE(n >= 1, MESH_MOE_E_ARG, "hidden_product: bad size n=%lld",
              (long long)n);
  MOE_REQUIRE(!noise_out || uniform, MESH_MOE_E_ARG,
              "hidden_product: noise_out without uniform");
  MOE_REQUIRE(!uniform || (keep_prob > 0.f && keep_prob <= 1.f), MESH_MOE_E_ARG,
              "hidden_product: keep_prob %g outside (0, 1]", (double)keep_prob);
  if (!factor && !uniform) return 0;
  hipStream_t st = (hipStream_t)stream;
  const int blocks = (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (x8_applies(n, dtype, h, factor, uniform, noise_out)) {
    const float keep = round_bf16_host(keep_prob);
    hidden_product_bf16x8_kernel<<<elementwise_blocks(n / 8), 256, 0, st>>>(
        (uint4*)h, (const uint4*)factor, (const uint4*)uniform, keep,
        round_bf16_host(1.f / keep), (uint4*)noise_out, n / 8);
  } else if (dtype == MESH_MOE_F32) {
    hidden_product_kernel<float><<<blocks, 256, 0, st>>>(
        (float*)h, (const float*)factor, (const float*)uniform, keep_prob,
        1.f / keep_prob, (float*)noise_out, n);
  } else {
    // the threshold and 1 / keep_prob are scalars of the activation dtype
    const float keep = round_bf16_host(keep_prob);
    hidden_product_kernel<bf16_t><<<blocks, 256, 0, st>>>(
        (bf16_t*)h, (const bf16_t*)factor, (const bf16_t*)uniform, keep,
        round_bf16_host(1.f / keep), (bf16_t*)noise_out, n);
  }
  MOE_CHECK_LAUNCH("hidden_product");
  return 0;
}

extern "C" int mesh_moe_activation(const void* pre, void* out, int64_t n,
                                   int activation, int dtype, void* stream) {
  MOE_REQUIRE(pre && out, MESH_MOE_E_ARG, "activation: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG, "activation: bad dtype %d",
              dtype);
  MOE_REQUIRE(n >= 1, MESH_MOE_E_ARG, "activation: bad size n=%lld",
              (long long)n);
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "activation: unknown activation %d", activation);
  hipStream_t st = (hipStream_t)stream;
  const int blocks = (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (x8_applies(n, dtype, pre, out, nullptr))
    activation_bf16x8_kernel<<<elementwise_blocks(n / 8), 256, 0, st>>>(
        (const uint4*)pre, (uint4*)out, n / 8, activation);
  else if (dtype == MESH_MOE_F32)
    activation_copy_kernel<float><<<blocks, 256, 0, st>>>(
        (const float*)pre, (float*)out, n, activation);
  else
    activation_copy_kernel<bf16_t><<<blocks, 256, 0, st>>>(
        (const bf16_t*)pre, (bf16_t*)out, n, activation);
  MOE_CHECK_LAUNCH("activation");
  return 0;
}

extern "C" int mesh_moe_activation_backward(const void* dh, const void* pre,
                                            const void* factor, void* dpre,
                                            int64_t n, int activation,
                                            int dtype, void* stream) {
  MOE_REQUIRE(dh && pre && dpre, MESH_MOE_E_ARG,
              "activation_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "activation_backward: bad dtype %d", dtype);
  MOE_REQUIRE(n >= 1, MESH_MOE_E_ARG, "activation_backward: bad size n=%lld",
              (long long)n);
  MOE_REQUIRE(activation >= MESH_MOE_ACT_LINEAR &&
                  activation <= MESH_MOE_ACT_SWISH,
              MESH_MOE_E_ARG, "activation_backward: unknown activation %d",
              activation);
  hipStream_t st = (hipStream_t)stream;
  const int blocks = (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (dtype == MESH_MOE_F32)
    activation_backward_kernel<float><<<blocks, 256, 0, st>>>(
        (const float*)dh, (const float*)pre, (const float*)factor,
        (float*)dpre, n, activation);
  else if (n % 8 == 0 &&
           (((uintptr_t)dh | (uintptr_t)pre | (uintptr_t)factor |
             (uintptr_t)dpre) % 16) == 0) {
    const int64_t n8 = n / 8;
    const int vb = (int)((n8 + 255) / 256 < 16384 ? (n8 + 255) / 256 : 16384);
    activation_backward_bf16x8_kernel<<<vb, 256, 0, st>>>(
        (const uint4*)dh, (const uint4*)pre, (const uint4*)factor, (uint4*)dpre,
        n8, activation);
  } else
    activation_backward_kernel<bf16_t><<<blocks, 256, 0, st>>>(
        (const bf16_t*)dh, (const bf16_t*)pre, (const bf16_t*)factor,
        (bf16_t*)dpre, n, activation);
  MOE_CHECK_LAUNCH("activation_backward");
  return 0;
}

extern "C" size_t mesh_moe_expert_linear_backward_workspace_bytes(int E, int R,
                                                                  int K, int N,
                                                                  int dtype) {
  if (E < 1 || R < 1 || K < 1 || N < 1 || !valid_dtype(dtype)) return 0;
  return ((size_t)E * R * K + (size_t)E * R * N) * dtype_size(dtype) + 2 * 256;
}

extern "C" int mesh_moe_expert_linear_backward(
    const void* a, const void* dy, const void* w, void* da, void* dw,
    const void* da_relu_mask, int E, int R, int K, int N, int dtype,
    void* workspace, size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(a && dy && w && dw && workspace, MESH_MOE_E_ARG,
              "expert_linear_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "expert_linear_backward: bad dtype %d", dtype);
  MOE_REQUIRE(E >= 1 && R >= 1 && K >= 1 && N >= 1, MESH_MOE_E_ARG,
              "expert_linear_backward: bad sizes E=%d R=%d K=%d N=%d", E, R, K,
              N);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_expert_linear_backward_workspace_bytes(E, R, K, N,
                                                                  dtype),
              MESH_MOE_E_ARG, "expert_linear_backward: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (da != nullptr) {
    // da = dy . w^T  (w in its variable layout [E, K, N] is K-contiguous here);
    // a ReLU mask rides on the stores of this GEMM where its kernel can
    bool masked = false;
    rc = grouped_gemm(dy, w, da, E, R, K, N, MESH_MOE_ACT_LINEAR, dtype, st,
                      da_relu_mask, &masked);
    if (rc != 0) return rc;
    if (da_relu_mask != nullptr && !masked) {
      rc = launch_hidden_grad(da, da_relu_mask, nullptr, true,
                              (int64_t)E * R * K, dtype, st);
      if (rc != 0) return rc;
    }
  }
  // dw [E, K, N] = a^T . dy: the reduction runs over the rows of both operands
  if (kmajor_path_applies(a, dy, dw, K, N, R, dtype))
    return launch_ring_kmajor((const bf16_t*)a, (const bf16_t*)dy, (bf16_t*)dw,
                              E, K, N, R, st);
  const size_t es = dtype_size(dtype);
  auto up = [](uintptr_t v) { return (v + 255) & ~(uintptr_t)255; };
  unsigned char* tr_a = (unsigned char*)up((uintptr_t)workspace);
  unsigned char* tr_dy =
      (unsigned char*)up((uintptr_t)(tr_a + (size_t)E * R * K * es));
  rc = mesh_moe_pack_weights(a, tr_a, E, R, K, dtype, dtype, stream);
  if (rc != 0) return rc;
  rc = mesh_moe_pack_weights(dy, tr_dy, E, R, N, dtype, dtype, stream);
  if (rc != 0) return rc;
  return grouped_gemm(tr_a, tr_dy, dw, E, K, N, R, MESH_MOE_ACT_LINEAR, dtype,
                      st);
}

// Elements of the scratch mesh_moe_expert_ffn_backward needs: dh [E,R,H], one
// [E,H,R] transpose buffer (h^T, then dh^T) and one [E,max(M,N),R] buffer
// (dy^T, then expert_in^T).
static size_t ffn_backward_elems(int E, int R, int M, int H, int N) {
  const size_t mn = (size_t)(M > N ? M : N);
  return (size_t)E * R * H * 2 + (size_t)E * R * mn;
}

extern "C" size_t mesh_moe_expert_ffn_backward_workspace_bytes(int E, int R,
                                                               int M, int H,
                                                               int N,
                                                               int dtype) {
  if (E < 1 || R < 1 || M < 1 || H < 1 || N < 1 || !valid_dtype(dtype))
    return 0;
  return ffn_backward_elems(E, R, M, H, N) * dtype_size(dtype) + 3 * 256;
}

extern "C" int mesh_moe_expert_ffn_backward(
    const void* expert_in, const void* h, const void* dy, const void* wi,
    const void* wo, const void* dh_scale, float dh_keep_prob,
    void* dexpert_in, void* dwi, void* dwo, int E, int R,
    int M, int H, int N, int activation, int dtype, void* workspace,
    size_t workspace_bytes, void* stream) {
  MOE_REQUIRE(expert_in && h && dy && wi && wo && dexpert_in && dwi && dwo &&
                  workspace, MESH_MOE_E_ARG,
              "expert_ffn_backward: null pointer");
  MOE_REQUIRE(valid_dtype(dtype), MESH_MOE_E_ARG,
              "expert_ffn_backward: bad dtype %d", dtype);
  MOE_REQUIRE(E >= 1 && R >= 1 && M >= 1 && H >= 1 && N >= 1, MESH_MOE_E_ARG,
              "expert_ffn_backward: bad sizes E=%d R=%d M=%d H=%d N=%d", E, R,
              M, H, N);
  MOE_REQUIRE(activation == MESH_MOE_ACT_RELU ||
                  activation == MESH_MOE_ACT_LINEAR, MESH_MOE_E_UNSUPPORTED,
              "expert_ffn_backward: only relu and linear experts (got %d): the "
              "other activations need the pre-activation, which is not kept",
              activation);
  MOE_REQUIRE(dh_keep_prob >= 0.f && dh_keep_prob <= 1.f, MESH_MOE_E_ARG,
              "expert_ffn_backward: dh_keep_prob=%g outside [0, 1] (0: no "
              "dropout, or a noise tensor alone describes it)",
              (double)dh_keep_prob);
  MOE_REQUIRE(workspace_bytes >= mesh_moe_expert_ffn_backward_workspace_bytes(
                                     E, R, M, H, N, dtype),
              MESH_MOE_E_ARG, "expert_ffn_backward: workspace too small");
  const size_t es = dtype_size(dtype);
  auto up = [](uintptr_t v) { return (v + 255) & ~(uintptr_t)255; };
  unsigned char* dh = (unsigned char*)up((uintptr_t)workspace);
  unsigned char* tr_h = (unsigned char*)up((uintptr_t)(dh + (size_t)E * R * H * es));
  unsigned char* tr_mn = (unsigned char*)up((uintptr_t)(tr_h + (size_t)E * R * H * es));
  hipStream_t st = (hipStream_t)stream;
  int rc;
  // dh = dy . wo^T  (wo in its variable layout [E, H, N] is K-contiguous here)
  // (the ReLU mask rides on the stores of this GEMM where its kernel can)
  // With a dropout whose keep probability is known, a ReLU expert's noise need
  // not be read: where the stored activation is positive the element was kept
  // and its noise is 1 / keep_prob (as mesh_moe_hidden_product rounds it).
  const bool relu_act = activation == MESH_MOE_ACT_RELU;
  const bool noise_by_mask =
      relu_act && dh_keep_prob > 0.f && dh_keep_prob < 1.f;
  // 1 / keep_prob as mesh_moe_hidden_product has it
  const float mask_scale =
      !noise_by_mask ? 1.f
      : dtype == MESH_MOE_BF16
          ? round_bf16_host(1.f / round_bf16_host(dh_keep_prob))
          : 1.f / dh_keep_prob;
  bool masked = false;
  rc = grouped_gemm(dy, wo, dh, E, R, H, N, MESH_MOE_ACT_LINEAR, dtype, st,
                    relu_act && (!dh_scale || noise_by_mask) ? h : nullptr,
                    &masked, mask_scale);
  if (rc != 0) return rc;
  if (!masked && (relu_act || dh_scale)) {
    rc = launch_hidden_grad(dh, h, noise_by_mask ? nullptr : dh_scale, relu_act,
                            (int64_t)E * R * H, dtype, st, mask_scale);
    if (rc != 0) return rc;
  }
  // dexpert_in = dh . wi^T  (wi in its variable layout [E, M, H])
  rc = grouped_gemm(dh, wi, dexpert_in, E, R, M, H, MESH_MOE_ACT_LINEAR, dtype,
                    st);
  if (rc != 0) return rc;
  // dwo [E, H, N] = h^T . dy and dwi [E, M, H] = expert_in^T . dh: the
  // reduction runs over token rows, the outermost index of both operands
  if (kmajor_path_applies(h, dy, dwo, H, N, R, dtype) &&
      kmajor_path_applies(expert_in, dh, dwi, M, H, R, dtype)) {
    rc = launch_ring_kmajor((const bf16_t*)h, (const bf16_t*)dy, (bf16_t*)dwo,
                            E, H, N, R, st);
    if (rc != 0) return rc;
    return launch_ring_kmajor((const bf16_t*)expert_in, (const bf16_t*)dh,
                              (bf16_t*)dwi, E, M, H, R, st);
  }
  // otherwise: both operands transposed to token-contiguous copies first
  rc = mesh_moe_pack_weights(h, tr_h, E, R, H, dtype, dtype, stream);
  if (rc != 0) return rc;
  rc = mesh_moe_pack_weights(dy, tr_mn, E, R, N, dtype, dtype, stream);
  if (rc != 0) return rc;
  rc = grouped_gemm(tr_h, tr_mn, dwo, E, H, N, R, MESH_MOE_ACT_LINEAR, dtype,
                    st);
  if (rc != 0) return rc;
  // dwi [E, M, H] = expert_in^T . dh
  rc = mesh_moe_pack_weights(expert_in, tr_mn, E, R, M, dtype, dtype, stream);
  if (rc != 0) return rc;
  rc = mesh_moe_pack_weights(dh, tr_h, E, R, H, dtype, dtype, stream);
  if (rc != 0) return rc;
  return grouped_gemm(tr_mn, tr_h, dwi, E, M, H, R, MESH_MOE_ACT_LINEAR, dtype,
                      st);
}

// ---------------------------------------------------------------------------
// Backward of the expert feed-forward on COMPACTED rows (the row order of
// mesh_moe_compact_expert_ffn): the two GEMMs whose result has token rows
// (dh, dexpert_in) compute only the row tiles that hold occupied slots, the
// two weight-gradient GEMMs reduce over every expert's occupied rows only.
// ---------------------------------------------------------------------------
static bool compact_backward_applies(int G, int E, int C, int M, int H, int N) {
  if (G < 1 || E < 1 || E > 1024 || C < 1 || M < 1 || H < 1 || N < 1)
    return false;
  const int64_t rows = (int64_t)G * C;
  if (rows > 0x7fffffffLL) return false;
  const int R = (int)rows;
  return ring_path_applies(R, H, N) && ring_path_applies(R, M, H) &&
         kmajor_path_applies(nullptr, nullptr, nullptr, H, N, R,
                             MESH_MOE_BF16) &&
         kmajor_path_applies(nullptr, nullptr, nullptr, M, H, R, MESH_MOE_BF16);
}

extern "C" size_t mesh_moe_compact_expert_ffn_backward_workspace_bytes(
    int G, int E, int C, int M, int H, int N) {
  if (!compact_backward_applies(G, E, C, M, H, N)) return 0;
  const size_t R = (size_t)G * C;
  const size_t tm = (R + RingCfg::BM - 1) / RingCfg::BM;
  const size_t tiles = (size_t)E * tm *
                       ((size_t)(H + RingCfg::BN - 1) / RingCfg::BN +
                        (size_t)(M + RingCfg::BN - 1) / RingCfg::BN);
  return sizeof(bf16_t) * (size_t)E * R * H +
         sizeof(int32_t) * ((size_t)E + tiles + 2 * 64) + 5 * 256;
}

extern "C" int mesh_moe_compact_expert_ffn_backward(
    const void* expert_in, const void* h, const void* dy, const void* wi,
    const void* wo, const void* dh_scale, float dh_keep_prob,
    const int32_t* fill, const int32_t* row_offsets, void* dexpert_in,
    void* dwi, void* dwo, int G, int E, int C, int M, int H, int N,
    int activation, int dtype, void* workspace, size_t workspace_bytes,
    void* stream) {
  MOE_REQUIRE(expert_in && h && dy && wi && wo && fill && row_offsets &&
                  dexpert_in && dwi && dwo && workspace, MESH_MOE_E_ARG,
              "compact_expert_ffn_backward: null pointer");
  MOE_REQUIRE(G >= 1 && E >= 1 && C >= 1 && M >= 1 && H >= 1 && N >= 1,
              MESH_MOE_E_ARG, "compact_expert_ffn_backward: bad sizes");
  MOE_REQUIRE(activation == MESH_MOE_ACT_RELU ||
                  activation == MESH_MOE_ACT_LINEAR, MESH_MOE_E_UNSUPPORTED,
              "compact_expert_ffn_backward: only relu and linear experts (got "
              "%d)", activation);
  MOE_REQUIRE(dh_keep_prob >= 0.f && dh_keep_prob <= 1.f, MESH_MOE_E_ARG,
              "compact_expert_ffn_backward: dh_keep_prob=%g outside [0, 1]",
              (double)dh_keep_prob);
  MOE_REQUIRE(dtype == MESH_MOE_BF16 &&
                  compact_backward_applies(G, E, C, M, H, N) &&
                  (((uintptr_t)expert_in | (uintptr_t)h | (uintptr_t)dy |
                    (uintptr_t)wi | (uintptr_t)wo | (uintptr_t)dexpert_in |
                    (uintptr_t)dwi | (uintptr_t)dwo) % 16 == 0),
              MESH_MOE_E_UNSUPPORTED,
              "compact_expert_ffn_backward: needs bf16, at most 1024 experts "
              "and shapes the 256 x 256 direct-to-LDS kernels take (rows=%lld "
              "M=%d H=%d N=%d)", (long long)G * C, M, H, N);
  MOE_REQUIRE(workspace_bytes >=
                  mesh_moe_compact_expert_ffn_backward_workspace_bytes(
                      G, E, C, M, H, N),
              MESH_MOE_E_ARG, "compact_expert_ffn_backward: workspace too small");
  hipStream_t st = (hipStream_t)stream;
  const int R = G * C;
  auto up = [](uintptr_t q) { return (q + 255) & ~(uintptr_t)255; };
  bf16_t* dh = (bf16_t*)up((uintptr_t)workspace);
  int32_t* rows_used = (int32_t*)up((uintptr_t)(dh + (size_t)E * R * H));
  const int tiles_m = (R + RingCfg::BM - 1) / RingCfg::BM;
  const int tn_h = (H + RingCfg::BN - 1) / RingCfg::BN;
  const int tn_m = (M + RingCfg::BN - 1) / RingCfg::BN;
  int32_t* list_h = (int32_t*)up((uintptr_t)(rows_used + E)) + 64;
  int32_t* list_m =
      (int32_t*)up((uintptr_t)(list_h + (size_t)E * tiles_m * tn_h)) + 64;
  rows_used_kernel<<<(E + 255) / 256, 256, 0, st>>>(fill, row_offsets,
                                                    rows_used, G, E);
  MOE_CHECK_LAUNCH("compact_expert_ffn_backward (rows used)");
  tile_list_kernel<<<1, 1024, 0, st>>>(rows_used, list_h, E, tiles_m, tn_h,
                                       RingCfg::BM);
  MOE_CHECK_LAUNCH("compact_expert_ffn_backward (tile list 1)");
  tile_list_kernel<<<1, 1024, 0, st>>>(rows_used, list_m, E, tiles_m, tn_m,
                                       RingCfg::BM);
  MOE_CHECK_LAUNCH("compact_expert_ffn_backward (tile list 2)");
  // dh = dy . wo^T on the listed row tiles, the ReLU mask on its stores (the
  // rows of a listed tile past the expert's occupied ones have h = 0 and
  // dy = 0)
  // (a ReLU expert's dropout noise follows from the stored activation: see
  // mesh_moe_expert_ffn_backward)
  const bool noise_by_mask = activation == MESH_MOE_ACT_RELU &&
                             dh_keep_prob > 0.f && dh_keep_prob < 1.f;
  const float mask_scale =
      noise_by_mask ? round_bf16_host(1.f / round_bf16_host(dh_keep_prob)) : 1.f;
  const bool mask_on_stores =
      activation == MESH_MOE_ACT_RELU && (!dh_scale || noise_by_mask);
  int rc = launch_ring(
      (const bf16_t*)dy, (const bf16_t*)wo, dh, E, R, H, N, false, st, nullptr,
      nullptr, mask_on_stores ? (const bf16_t*)h : nullptr, list_h, mask_scale);
  if (rc != 0) return rc;
  if (dh_scale != nullptr && !mask_on_stores) {
    // the dropout's noise (and the ReLU mask) as a pass over the buffer, as in
    // mesh_moe_expert_ffn_backward; rows outside the listed tiles hold
    // unspecified values before and after
    rc = launch_hidden_grad(dh, h, dh_scale, activation == MESH_MOE_ACT_RELU,
                            (int64_t)E * R * H, dtype, st);
    if (rc != 0) return rc;
  }
  // dexpert_in = dh . wi^T on the listed row tiles
  rc = launch_ring(dh, (const bf16_t*)wi, (bf16_t*)dexpert_in, E, R, M, H,
                   false, st, nullptr, nullptr, nullptr, list_m);
  if (rc != 0) return rc;
  // dwo = h^T . dy and dwi = expert_in^T . dh over the occupied rows
  rc = launch_ring_kmajor((const bf16_t*)h, (const bf16_t*)dy, (bf16_t*)dwo, E,
                          H, N, R, st, rows_used);
  if (rc != 0) return rc;
  return launch_ring_kmajor((const bf16_t*)expert_in, dh, (bf16_t*)dwi, E, M,
                            H, R, st, rows_used);
}
