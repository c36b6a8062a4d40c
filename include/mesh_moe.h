/*
 * mesh_moe.h -- C ABI of libmesh_moe_hip.so: the top-2 Mixture-of-Experts
 * forward path of Mesh TensorFlow (mesh_tensorflow/transformer/moe.py) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller unless the
 *     parameter name ends in _host; the library never allocates or frees;
 *   - every call is asynchronous on the hipStream_t passed as `stream`
 *     (a void* here so that C callers need no HIP headers; 0 = null stream);
 *   - return value 0 = launched, negative = rejected before any launch
 *     (MESH_MOE_E_*); mesh_moe_last_error() gives the reason for the calling
 *     thread's last rejected call;
 *   - all tensors are dense row-major with the shapes written in brackets.
 *
 * Each entry point names the part of the reference it replaces
 * (file:line under the reference tree).  The reference itself has no FFI: it
 * lowers the layer to ~100 TensorFlow ops through MeshImpl.slicewise
 * (mesh_tensorflow/ops.py:1019-1030); these functions are what a MeshImpl's
 * slice function binds instead.
 */
#ifndef MESH_MOE_H_
#define MESH_MOE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MESH_MOE_ABI_VERSION 34

/* element types of activations / weights */
#define MESH_MOE_F32 0
#define MESH_MOE_BF16 1

/* moe_second_policy_* (transformer/moe.py:1452-1467) */
#define MESH_MOE_SECOND_ALL 0
#define MESH_MOE_SECOND_NONE 1
#define MESH_MOE_SECOND_THRESHOLD 2
#define MESH_MOE_SECOND_RANDOM 3

/* expert activation (mesh_tensorflow/ops.py:1818-1921) */
#define MESH_MOE_ACT_LINEAR 0
#define MESH_MOE_ACT_RELU 1
#define MESH_MOE_ACT_GELU 2
#define MESH_MOE_ACT_SIGMOID 3
#define MESH_MOE_ACT_TANH 4
#define MESH_MOE_ACT_SWISH 5

/* error codes */
#define MESH_MOE_E_ARG (-1)        /* bad argument (null, size, enum)        */
#define MESH_MOE_E_UNSUPPORTED (-2) /* shape outside what the kernels handle */
#define MESH_MOE_E_HIP (-3)        /* a HIP runtime call failed              */

int mesh_moe_abi_version(void);
const char* mesh_moe_last_error(void);

/*
 * CRC-32C (Castagnoli) of data[0, n) continued from `crc` (0 to start): the
 * checksum TensorFlow's tensor-bundle checkpoint files carry for every table
 * block and every tensor (tensorflow/core/lib/hash/crc32c.h `Extend`; TensorFlow
 * is the reference's dependency and is not vendored in it).  Host code; `data`
 * is a host pointer.  The reference reaches those files through tf.train
 * (mesh_tensorflow/transformer/utils.py:947-972, tf.train.init_from_checkpoint).
 */
uint32_t mesh_moe_crc32c(uint32_t crc, const void* data, size_t n);

/*
 * Router projection: logits[b,t,e] = sum_m float(x[b,t,m]) * float(w[b,m,e])
 * (+ bias[e] if bias != NULL), float32 accumulate.
 * Replaces the `mtf.layers.dense(gate_inputs, experts_dim, use_bias=False)`
 * einsum of _top_2_gating (transformer/moe.py:1384-1390; layers.py:129-208).
 * batch > 1 is the inner level of the hierarchical layer, where every outer
 * expert has its own router (outer_expert_dims, moe.py:743-753).
 *   x [batch, tokens, M] dtype; w [batch, M, E] dtype; logits [batch,tokens,E]
 *   w_packed [batch, E, M] dtype or NULL: the same weights K-contiguous (see
 *   mesh_moe_pack_weights).  When given (bf16, M % 64 == 0, E % 4 == 0) the
 *   projection runs on the matrix cores and is bound by reading x once.
 * `bias` is a benchmark hook (skewed-routing stress); the reference has none.
 */
int mesh_moe_router_logits(const void* x, const void* w, const void* w_packed,
                           const float* bias, float* logits, int batch,
                           int64_t tokens, int M, int E, int dtype,
                           void* stream);

/* Bytes of scratch mesh_moe_top2_gating needs for (G, S, E). */
size_t mesh_moe_gating_workspace_bytes(int G, int S, int E);

/*
 * Top-2 gating from router logits: softmax, first/second expert, gate
 * normalisation, second-place policy, per-group capacity positions with
 * overflow drop, and the load-balancing loss.
 * Replaces _top_2_gating after the router projection
 * (transformer/moe.py:1391-1496, :1508) -- softmax ops.py:5493-5541, top_1
 * ops.py:4937-4940, cumsum ops.py:2761-2781 -- without building the dense
 * [G,S,E,C] combine/dispatch tensors (moe.py:1499-1511): the per-token record
 * below carries the same information.
 *   logits      [G,S,E] float32
 *   importance  [G,S] of importance_dtype, or NULL  (moe.py:1401-1411).
 *               With importance_from_slot_gate != 0 the array holds the slot
 *               weights w written by mesh_moe_dispatch and the importance is
 *               0.5 * ((w > 0.5) + (w > 0))  (hierarchical layer, moe.py:725-727)
 *   second_uniform [G,S] float32 U(0,1) samples, required for policy RANDOM
 *   idx  [G,S,2] int32   expert of first / second choice
 *   pos  [G,S,2] int32   position_in_expert_k (raw; >= C when dropped)
 *   gate [G,S,2] float32 normalised gate_k * mask_k_flat (moe.py:1485,:1494)
 *   kept [G,S,2] uint8   mask_k_flat
 *   fill [G,E]   int32   occupied slots of each expert after both passes
 *   loss [1]     float32 balancing loss before moe_loss_coef (moe.py:1420-1442)
 * Limits: 2 <= E <= 512, S <= 16384, C >= 1.
 */
int mesh_moe_top2_gating(const float* logits, const void* importance,
                         int importance_dtype, int importance_from_slot_gate,
                         const float* second_uniform, int G, int S, int E,
                         int C, int policy,
                         double threshold, int use_second_place_loss,
                         int num_microbatches, int32_t* idx, int32_t* pos,
                         float* gate, uint8_t* kept, int32_t* fill,
                         float* loss, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Size of the scratch array mesh_moe_top2_gating_static_scratch keeps on
 * every GPU the library runs on, until the process ends. */
#define MESH_MOE_STATIC_SCRATCH_BYTES (4u << 20)

/*
 * mesh_moe_top2_gating without the workspace argument.  It has no counterpart
 * in the reference: it exists for callers that cannot allocate device memory
 * or carry a workspace around (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  The scratch memory the kernels
 * need (per-block partial sums of the loss, per-group sums) lives in an array
 * of MESH_MOE_STATIC_SCRATCH_BYTES that is part of the library's device code;
 * its address is looked up once per device, on the first call made with that
 * device current.  The call allocates and frees nothing.
 * Same arguments, results and limits as mesh_moe_top2_gating, plus:
 * MESH_MOE_E_UNSUPPORTED (nothing launched) when
 * mesh_moe_gating_workspace_bytes(G, S, E) > MESH_MOE_STATIC_SCRATCH_BYTES.
 * Every call on a GPU shares that GPU's array: two calls that overlap in time
 * on one GPU (different streams, or different threads) race; serialise them.
 * Nothing in the array has to survive between calls or start at zero.
 */
int mesh_moe_top2_gating_static_scratch(
    const float* logits, const void* importance, int importance_dtype,
    int importance_from_slot_gate, const float* second_uniform, int G, int S,
    int E, int C, int policy, double threshold, int use_second_place_loss,
    int num_microbatches, int32_t* idx, int32_t* pos, float* gate,
    uint8_t* kept, int32_t* fill, float* loss, void* stream);

/*
 * Router projection and top-2 gating in one call and ONE kernel launch: what
 * _top_2_gating does from `to_float(inputs)` to the per-token assignment
 * (transformer/moe.py:1384-1496).  The logits stay in LDS between the
 * matrix-core projection and the softmax / top-2 step (they are written to
 * `logits` [G,S,E] only if it is not NULL); every block ranks the choices of
 * its 128 tokens with wavefront ballots and publishes per-expert counts, and
 * the block of a group that finishes last turns them into capacity positions,
 * `fill` and the group's loss term (no block waits for another).  Arguments
 * are those of mesh_moe_router_logits (packed weights only) followed by those
 * of mesh_moe_top2_gating; batch * tokens == G * S and each weight set covers
 * whole groups.  The workspace may hold anything on entry.
 * Returns MESH_MOE_E_UNSUPPORTED (nothing launched) unless dtype is bf16,
 * M % 64 == 0, E % 4 == 0, E <= 128 and S % 128 == 0; callers then use the two
 * separate entry points.
 */
int mesh_moe_router_top2_gating(
    const void* x, const void* w_packed, const float* bias, float* logits,
    int batch, int64_t tokens, int M, int dtype, const void* importance,
    int importance_dtype, int importance_from_slot_gate,
    const float* second_uniform, int G, int S, int E, int C, int policy,
    double threshold, int use_second_place_loss, int num_microbatches,
    int32_t* idx, int32_t* pos, float* gate, uint8_t* kept, int32_t* fill,
    float* loss, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Switch (top-1) gating from router logits: softmax, arg-max expert, raw
 * probability as the gate, per-group capacity positions with overflow drop,
 * load-balancing loss and (optionally) the router z-loss.
 * Replaces _switch_gating and _switch_max_gating after the router projection
 * (transformer/moe.py:1207-1306, :976-1051; z-loss :1253-1266).  The policies
 * "input_dropout" / "input_jitter" change the projection's input, which is
 * the caller's business; policy "sample" passes choice_logits.
 * The per-token record has the layout of mesh_moe_top2_gating with the second
 * choice never kept (kept[..,1] = 0, gate[..,1] = 0), so mesh_moe_dispatch and
 * mesh_moe_combine apply unchanged.
 *   choice_logits [G,S,E] float32 or NULL: when given, a token's expert is
 *               the first arg-max of its row here instead of the arg-max of
 *               the probabilities, and the gate is the probability of that
 *               expert (policy "sample", moe.py:1213-1216: the caller passes
 *               logits + Gumbel noise * temperature, ops.py:5070-5086)
 *   importance [G,S] of importance_dtype or NULL: only tokens with
 *               importance == 1 are routed (moe.py:1226-1231)
 *   slots_by_gate  0: an expert's slots go to its choosers in token order,
 *               overflow dropped (_switch_gating, moe.py:1268-1291);
 *               1: to the `C` choosers with the largest gate, slot c holding
 *               the (c+1)-th largest, equal gates in token order
 *               (_switch_max_gating, transformer/moe.py:1033-1039, the top_k
 *               of ops.py:4934-4942); pos then is that rank
 *   use_z_loss != 0 adds z_loss_coef * sum_t(logsumexp_t^2 * (imp_t == 1)) /
 *               (#(imp == 1) * num_microbatches); the caller passes it only
 *               when training with hparams.moe_z_loss set
 *   loss [1]  float32, before moe_loss_coef
 * Limits as mesh_moe_top2_gating; workspace from
 * mesh_moe_gating_workspace_bytes.
 */
int mesh_moe_switch_gating(const float* logits, const float* choice_logits,
                           const void* importance, int importance_dtype, int G,
                           int S, int E, int C,
                           int slots_by_gate, int use_z_loss,
                           double z_loss_coef,
                           int num_microbatches, int32_t* idx, int32_t* pos,
                           float* gate, uint8_t* kept, int32_t* fill,
                           float* loss, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * Router projection + switch gating in one call (transformer/moe.py:1200-1306);
 * the switch counterpart of mesh_moe_router_top2_gating, same shape limits and
 * the same MESH_MOE_E_UNSUPPORTED convention.
 */
int mesh_moe_router_switch_gating(
    const void* x, const void* w_packed, const float* bias, float* logits,
    int batch, int64_t tokens, int M, int dtype, const void* importance,
    int importance_dtype, int G, int S, int E, int C, int slots_by_gate,
    int use_z_loss, double z_loss_coef, int num_microbatches, int32_t* idx,
    int32_t* pos, float* gate, uint8_t* kept, int32_t* fill, float* loss,
    void* workspace, size_t workspace_bytes, void* stream);

/*
 * Dispatch: expert_in[e,g,c,:] = x[g,s,:] for the token holding slot (e,g,c),
 * zero rows for empty slots.  Replaces the one-hot dispatch einsum
 * (transformer/moe.py:443-447; a slot whose activation-dtype gate is exactly
 * zero is not dispatched, moe.py:1510-1511).
 *   x [G,S,M] dtype; expert_in [E,G,C,M] dtype
 *   slot_gate [E,G,C] float32 or NULL: the activation-dtype combine weight of
 *   the token in each slot (0 for empty slots) = reduce_sum(combine_tensor)
 *   over the group-size dim, which the hierarchical layer turns into the
 *   importance of the inner level (moe.py:724-727).
 */
int mesh_moe_dispatch(const void* x, const int32_t* idx, const int32_t* pos,
                      const float* gate, const uint8_t* kept,
                      const int32_t* fill, void* expert_in, float* slot_gate,
                      int G, int S, int E, int C, int M, int dtype,
                      void* stream);

/*
 * Expert weights are consumed in a K-contiguous ("packed") layout:
 *   packed[e][n][k] = (dtype) src[e][k][n]
 * mesh_moe_pack_weights converts the reference's variable layout
 * (`wi/kernel` [experts, d_model, expert_hidden], `wo/kernel`
 * [experts, expert_hidden, d_model], transformer/moe.py:469-486,
 * layers.py:239-251) and casts master dtype -> activation dtype, i.e. it is
 * the copy_master_to_slices + cast of Variable.lower (ops.py:4039-4051,
 * placement_mesh_impl.py:67-157) for this MeshImpl.
 *   src [E,K,N] src_dtype; dst [E,N,K] dst_dtype
 */
int mesh_moe_pack_weights(const void* src, void* dst, int E, int K, int N,
                          int src_dtype, int dst_dtype, void* stream);

/*
 * Expert feed-forward: h = act(expert_in . wi); y = h . wo, per expert,
 * float32 accumulate, h and y stored in dtype.  Replaces dense_product "wi" +
 * dense "wo" (transformer/moe.py:469-486; v2 :765-774).
 *   expert_in [E,R,M] dtype (R = rows per expert = groups * capacity)
 *   wi_packed [E,H,M] dtype; wo_packed [E,N,H] dtype  (see pack_weights)
 *   h [E,R,H] dtype (caller-provided scratch); y [E,R,N] dtype
 * bf16 with M and H multiples of 8 runs on the MFMA kernel; float32 and other
 * shapes run on a plain FMA tile kernel.
 */
int mesh_moe_expert_ffn(const void* expert_in, const void* wi_packed,
                        const void* wo_packed, void* h, void* y, int E, int R,
                        int M, int H, int N, int activation, int dtype,
                        void* stream);

/*
 * One expert projection: y = act(a . w) per expert, float32 accumulate -- the
 * grouped GEMM mesh_moe_expert_ffn runs twice.  Replaces a single
 * mtf.layers.dense with expert_dims (layers.py:129-208), e.g. the "q_wo" and
 * "k_wo" projections of the same hidden tensor when moe_use_experts_attention
 * is set (transformer/moe.py:482-520).
 *   a [E,R,K] dtype; w_packed [E,N,K] dtype (see pack_weights); y [E,R,N] dtype
 */
int mesh_moe_expert_linear(const void* a, const void* w_packed, void* y, int E,
                           int R, int K, int N, int activation, int dtype,
                           void* stream);

/*
 * What the layer does to the hidden tensor between the two expert einsums, in
 * place on n elements of `dtype`, each product rounded once:
 *   factor  != NULL: h *= factor -- one more factor of mtf.layers.dense_product
 *            (layers.py:256-295) when the expert activation is a list (gated
 *            units, transformer/moe.py:469-475)
 *   uniform != NULL: h *= noise, noise = (uniform < keep_prob) / keep_prob with
 *            keep_prob and the quotient rounded to `dtype` -- mtf.dropout
 *            (ops.py:5832-5872) under hparams.moe_dropout_rate
 *            (transformer/moe.py:477-479); uniform [n] dtype in [0, 1)
 *   noise_out [n] dtype or NULL: the noise, kept for the backward pass
 */
int mesh_moe_hidden_product(void* h, const void* factor, const void* uniform,
                            float keep_prob, void* noise_out, int64_t n,
                            int dtype, void* stream);

/* Bytes of scratch mesh_moe_dispatched_expert_ffn needs. */
size_t mesh_moe_dispatched_expert_ffn_workspace_bytes(int G, int E, int C,
                                                      int M);

/*
 * mesh_moe_dispatch + mesh_moe_expert_ffn in one call (the dispatch einsum
 * and the two expert einsums, transformer/moe.py:443-447 and :469-486) that
 * never writes expert_in: the first GEMM fetches each slot's token row straight from x
 * through a slot -> token map built from the routing record (empty slots and
 * kept choices whose gate rounds to 0 read a zero row).  Same h and y as the
 * two calls.  For callers that do not need expert_in afterwards (inference;
 * the backward reads it).  bf16 only, and only where the first GEMM
 * ([G*C, M] x [M, H] per expert) fits the 256 x 256 direct-to-LDS kernel;
 * otherwise MESH_MOE_E_UNSUPPORTED with nothing launched: make the two calls.
 *   x [G,S,M] dtype; idx, pos, gate, kept as written by the gating calls
 *   h [E,G*C,H], y [E,G*C,N] dtype
 */
int mesh_moe_dispatched_expert_ffn(
    const void* x, const int32_t* idx, const int32_t* pos, const float* gate,
    const uint8_t* kept, const void* wi_packed, const void* wo_packed, void* h,
    void* y, void* workspace, size_t workspace_bytes, int G, int S, int E, int C,
    int M, int H, int N, int activation, int dtype, void* stream);

/*
 * Combine: out[g,s,:] = w1 * y[idx1,g,pos1,:] + w2 * y[idx2,g,pos2,:] with
 * w_k the activation-dtype-rounded gate_k; zero for tokens with no kept
 * choice.  Replaces the combine einsum (transformer/moe.py:509-510).
 *   y [E,G,C,N] dtype; out [G,S,N] dtype
 */
int mesh_moe_combine(const void* y, const int32_t* idx, const int32_t* pos,
                     const float* gate, const uint8_t* kept, void* out, int G,
                     int S, int E, int C, int N, int dtype, void* stream);

/* Bytes of scratch mesh_moe_compact_expert_ffn needs. */
size_t mesh_moe_compact_expert_ffn_workspace_bytes(int G, int E, int C, int M,
                                                   int H, int N);

/*
 * mesh_moe_dispatched_expert_ffn on COMPACTED rows: the dispatch einsum and
 * the two expert einsums (transformer/moe.py:443-447, :469-486) for routers
 * that leave many slots empty (one choice per token with a capacity factor
 * above 1: _switch_gating, _ntlb_gating, transformer/moe.py:1176-1309,
 * :804-940).  The reference multiplies every slot row, occupied or not; here
 * expert e's occupied slots (groups in order, slots in order) become rows
 * 0 .. used_e - 1 of its row range in h and y, and only the 256-row tiles that
 * hold such rows are computed.  Rows beyond used_e hold unspecified values.
 *   fill [G,E] as written by the gating calls
 *   row_offsets [E,G] int32 (output): row of expert e's first slot of group
 *     g; slot (e, g, c) is row row_offsets[e][g] + c of h[e] / y[e] -- what
 *     mesh_moe_combine_compact takes
 *   hidden_uniform [E,G*C,H] dtype or NULL, keep_prob, noise_out [E,G*C,H]
 *     or NULL: the dropout of the hidden tensor between the two einsums
 *     (transformer/moe.py:477-479) as mesh_moe_hidden_product applies it; a
 *     slot's noise is the one at its compacted row
 * Otherwise as mesh_moe_dispatched_expert_ffn (same limits, both GEMMs must
 * fit the 256 x 256 kernel, E <= 1024, MESH_MOE_E_UNSUPPORTED otherwise).
 */
int mesh_moe_compact_expert_ffn(
    const void* x, const int32_t* idx, const int32_t* pos, const float* gate,
    const uint8_t* kept, const int32_t* fill, const void* wi_packed,
    const void* wo_packed, void* h, void* y, int32_t* row_offsets,
    const void* hidden_uniform, float keep_prob, void* noise_out,
    void* workspace, size_t workspace_bytes, int G, int S, int E, int C, int M,
    int H, int N, int activation, int dtype, void* stream);

/*
 * mesh_moe_combine (transformer/moe.py:509-510) reading y in the compacted
 * row order of mesh_moe_compact_expert_ffn: y [E, G*C, N], slot (e, g, c) at
 * row row_offsets[e][g] + c.
 */
int mesh_moe_combine_compact(const void* y, const int32_t* idx,
                             const int32_t* pos, const float* gate,
                             const uint8_t* kept, const int32_t* row_offsets,
                             void* out, int G, int S, int E, int C, int N,
                             int dtype, void* stream);

/*
 * "No token left behind" gating (_ntlb_gating, transformer/moe.py:804-940)
 * after the router projection: every token names its top_k experts
 * (mtf.top_k, ops.py:4964-5015); pass i offers the tokens no expert has
 * taken yet, in token order, to their i-th expert, which takes them while its
 * total stays within the capacity (moe.py:903-934).  A token is routed at
 * most once, with the raw softmax probability of the expert that took it as
 * the gate.  The record has the [G,S,2] layout of the other routers with the
 * second choice never kept, so dispatch, the FFN and combine apply unchanged;
 * idx[g,s,0] of a token nobody took is its first candidate.  The loss is
 * E^2 * mean(density_1_proxy * density_1) over [G,k,E] (and over the group dim
 * when `importance` is given, moe.py:845-860).  top_k <= 8.
 *   softmax_dtype: the dtype the reference runs this router's projection
 *   result and softmax in, i.e. the activation dtype -- _ntlb_gating alone
 *   has no to_float in front of its projection and casts only the
 *   probabilities to float32 (moe.py:825-836).  MESH_MOE_BF16: the logits
 *   (float32-accumulated) are rounded to bfloat16 and every op of
 *   mtf.softmax (ops.py:5493-5541: add, exp, reduce_sum, log, add, add, exp)
 *   rounds its result to bfloat16; the sum accumulates in float32 in index
 *   order and rounds once.  MESH_MOE_F32: float32 throughout.
 */
size_t mesh_moe_ntlb_workspace_bytes(int G, int S, int E, int top_k);
int mesh_moe_ntlb_gating(const float* logits, int softmax_dtype,
                         const void* importance,
                         int importance_dtype, int G, int S, int E, int C,
                         int top_k, int num_microbatches, int32_t* idx,
                         int32_t* pos, float* gate, uint8_t* kept,
                         int32_t* fill, float* loss, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * ---------------------------------------------------------------------------
 * Expert-selection ("expert choice") gating: every expert picks, per group,
 * the C tokens it likes best (_expert_selection_gating,
 * transformer/moe.py:1057-1173).  A token can sit in the slots of several
 * experts or of none, so the record is per slot:
 *   slot_token  [G,E,C] int32    token (index within the group) of each slot
 *   slot_weight [G,E,C] float32  its combine weight before the dtype cast
 *   tok_slot    [G,S,E] int16    slot the token holds at expert e, -1 if none
 * ---------------------------------------------------------------------------
 */

/* Bytes of scratch mesh_moe_expert_choice_gating needs. */
size_t mesh_moe_expert_choice_workspace_bytes(int G, int S, int E, int C);

/*
 * Gating from router logits (transformer/moe.py:1092-1147): -1e9 on the logits
 * of tokens with importance 0, softmax over the GROUP dim, per (group, expert)
 * the C largest probabilities in descending order with equal ones in token
 * order (top_k, ops.py:4934-4942), weights divided by max(#experts that chose
 * the token, 1) if `normalize`, and the loss
 * mean(mean_e(p)^2 * (importance == 1) * sum_s importance) * S.
 *   logits [G,S,E] float32; importance [G,S] of importance_dtype or NULL
 *   (NULL = all ones; the reference requires it, moe.py:1138-1140)
 *   loss [1] float32 before moe_loss_coef
 * Limits: C <= S <= 32768.
 */
int mesh_moe_expert_choice_gating(const float* logits, const void* importance,
                                  int importance_dtype, int G, int S, int E,
                                  int C, int normalize, int num_microbatches,
                                  int32_t* slot_token, float* slot_weight,
                                  int16_t* tok_slot, float* loss,
                                  void* workspace, size_t workspace_bytes,
                                  void* stream);

/*
 * ---------------------------------------------------------------------------
 * Training-time scalar summaries of the switch, switch-max, ntlb and
 * expert-selection routers: the values the reference hands to
 * mtf.scalar_summary while training (transformer/moe.py:865-880, :981,
 * :1010-1025, :1041-1046, :1149-1165, :1213, :1242-1257, :1259-1269,
 * :1285-1289), recomputed from the router's float32 logits and its routing
 * record.  _top_2_gating emits none.
 *   logits [G,S,E] float32 (the router's, after any input noise);
 *   softmax_dtype as for mesh_moe_ntlb_gating (bfloat16 only with router 2);
 *   importance [G,S] or NULL (all 1);
 *   router 1 = switch / switch_max (needs kept [G,S,2]), 2 = ntlb (top_k
 *   candidates per token), 3 = expert selection (needs tok_slot [G,S,E]);
 *   out, float32:
 *     [0] mean over tokens of sum_e -p log(p + 1e-9)   ("<name>/entropy");
 *         router 3: mean over (group, expert) of the same sum over the
 *         group's tokens, the softmax running over the group
 *     [1] mean over tokens of the largest probability  ("expert_gate",
 *         routers 1 and 2; before the importance mask, moe.py:979-981)
 *     [2] kept first choices / sum of importance        ("fraction_routed",
 *         router 1)
 *     [3] sum over importance-1 tokens of logsumexp(logits)^2 /
 *         (number of importance-1 tokens * num_microbatches)
 *                                                       ("<name>/z_loss")
 *     routers 1, 2: [4 + e], e < E: the share of expert e among the choices
 *         of importance-1 tokens (first choices; ntlb: all top_k candidates)
 *         ("experts/..", one summary per expert);
 *     router 3: [4 + s], s < S: E * C * the number of (group, expert) pairs
 *         whose expert took the token at position s ("group_token/..").
 *   out has 4 + E (routers 1, 2) or 4 + S (router 3) elements.  Sums over
 *   tokens run per block and then over the blocks in a fixed order: the same
 *   bits on every run;
 *   they agree with a sequential sum to float32 rounding.
 * ---------------------------------------------------------------------------
 */
size_t mesh_moe_router_summaries_workspace_bytes(int G, int S, int E);
int mesh_moe_router_summaries(const float* logits, int softmax_dtype,
                              const void* importance, int importance_dtype,
                              const uint8_t* kept, const int16_t* tok_slot,
                              int G, int S, int E, int C, int router,
                              int top_k, int num_microbatches, float* out,
                              void* workspace, size_t workspace_bytes,
                              void* stream);

/*
 * Dispatch by slot: expert_in[e,g,c,:] = x[g, slot_token[g,e,c], :]
 * (transformer/moe.py:443-447 with the one-hot dispatch tensor of :1105-1106,
 * which is 1 for every slot whatever its weight, :1169-1170).
 *   x [G,S,M] dtype; expert_in [E,G,C,M] dtype
 */
int mesh_moe_slot_dispatch(const void* x, const int32_t* slot_token,
                           void* expert_in, int G, int S, int E, int C, int M,
                           int dtype, void* stream);

/*
 * Combine by slot: out[g,s,:] = sum over the experts e that chose token s of
 * w * y[e,g,tok_slot[g,s,e],:], w the activation-dtype-rounded slot weight;
 * float32 accumulate in expert order, one rounding; zero rows for tokens
 * nobody chose (transformer/moe.py:509-510).
 *   y [E,G,C,N] dtype; out [G,S,N] dtype
 */
int mesh_moe_slot_combine(const void* y, const int16_t* tok_slot,
                          const float* slot_weight, void* out, int G, int S,
                          int E, int C, int N, int dtype, void* stream);

/*
 * Backward of the per-slot record (expert-selection gating).  The reference
 * gets these from mtf.gradients over the same einsums and over
 * _expert_selection_gating (transformer/moe.py:443-447, :509-510, :1094-1147):
 *
 * mesh_moe_slot_combine_backward: dy[e,g,c,:] = w * dout[g, token of the slot,:]
 *   with w the slot's combine weight as `dtype` holds it; dweight [G,E,C]
 *   float32 = <dout[g,token,:], y[e,g,c,:]>.
 * mesh_moe_slot_dispatch_backward: dx[g,s,:] = sum over the slots holding the
 *   token of dexpert_in[e,g,c,:] (+ dlogits[g,s,:] . w_gate^T when dlogits and
 *   w_gate_packed [E,M] are given), float32 accumulate, one rounding.
 *   w_gate [M,E] dtype or NULL: the router kernel in its variable layout; with
 *   it, as in mesh_moe_dispatch_backward, bf16 calls of the shapes named there
 *   take the router's share on the matrix cores.
 * mesh_moe_expert_choice_backward: d(logits) [G,S,E] float32 from dweight and
 *   from the gradient of the returned loss (d_loss [1] float32 on the device,
 *   loss_scale = moe_loss_coef): the softmax runs over the group's tokens per
 *   expert, a chosen probability is divided by the number of experts that chose
 *   the token (no gradient through that count), the loss goes through
 *   agg = mean_e p * (importance == 1).
 */
int mesh_moe_slot_combine_backward(const void* dout, const void* y,
                                   const int32_t* slot_token,
                                   const float* slot_weight, void* dy,
                                   float* dweight, int G, int S, int E, int C,
                                   int N, int dtype, void* stream);
int mesh_moe_slot_dispatch_backward(const void* dexpert_in,
                                    const int16_t* tok_slot,
                                    const float* dlogits,
                                    const void* w_gate_packed,
                                    const void* w_gate, void* dx, int G, int S,
                                    int E, int C, int M, int dtype,
                                    void* stream);
size_t mesh_moe_expert_choice_backward_workspace_bytes(int G, int S, int E);
int mesh_moe_expert_choice_backward(const float* logits, const void* importance,
                                    int importance_dtype,
                                    const int16_t* tok_slot,
                                    const float* dweight, const float* d_loss,
                                    double loss_scale, int G, int S, int E,
                                    int C, int normalize, int num_microbatches,
                                    float* dlogits, void* workspace,
                                    size_t workspace_bytes, void* stream);

/*
 * ---------------------------------------------------------------------------
 * Backward.  The reference has no hand-written backward for the layer:
 * mtf.gradients (mesh_tensorflow/ops.py:5254-5291) assembles it from the
 * gradients of the einsums and element-wise ops the layer is built from
 * (EinsumOperation.gradient ops.py:2846-2854, TopKOperation.gradient
 * ops.py:4916-4920, softmax ops.py:5493-5541).  The entry points below are
 * those einsum gradients with the one-hot tensors replaced by the routing
 * record.  Gradient tensors have the activation dtype; the gating runs in
 * float32 as in the forward pass.  Order of calls for one layer:
 * combine_backward, expert_ffn_backward, gating_backward,
 * router_backward_weights, dispatch_backward.
 * ---------------------------------------------------------------------------
 */

/*
 * Backward of the combine einsum (transformer/moe.py:509-510):
 *   dy[e,g,c,:]  = w * dout[g,s,:] for the token in slot (e,g,c), zero rows for
 *                  empty slots (w = its activation-dtype combine weight)
 *   dgate[g,s,k] = <dout[g,s,:], y[idx_k,g,pos_k,:]>, 0 where not kept
 *   dout [G,S,N] dtype; y, dy [E,G,C,N] dtype; dgate [G,S,2] float32
 */
int mesh_moe_combine_backward(const void* dout, const void* y,
                              const int32_t* idx, const int32_t* pos,
                              const float* gate, const uint8_t* kept,
                              const int32_t* fill, void* dy, float* dgate,
                              int G, int S, int E, int C, int N, int dtype,
                              void* stream);

/* Bytes of scratch mesh_moe_expert_ffn_backward needs. */
size_t mesh_moe_expert_ffn_backward_workspace_bytes(int E, int R, int M, int H,
                                                    int N, int dtype);

/*
 * Backward of the two expert einsums (transformer/moe.py:469-486), ReLU or
 * linear experts:
 *   dh = (dy . wo^T) * dh_scale * (h > 0);  dwo = h^T . dy
 *   dexpert_in = dh . wi^T;                 dwi = expert_in^T . dh
 *   expert_in [E,R,M], h [E,R,H] (as mesh_moe_expert_ffn left it, after the
 *   hidden dropout if there was one), dy [E,R,N]
 *   wi [E,M,H], wo [E,H,N]: the variables' own layout (NOT the packed one)
 *   dh_scale [E,R,H] dtype or NULL: the dropout noise mesh_moe_hidden_product
 *   wrote (transformer/moe.py:477-479)
 *   dh_keep_prob in [0, 1] (anything else is refused): the keep probability
 *   that noise was made with, or 0 if the caller does not know it or there
 *   was no dropout.  dh_scale NULL together with dh_keep_prob 0 (or 1) means
 *   that no dropout was applied in the forward pass.  With a value in (0, 1)
 *   ReLU experts do not read dh_scale, which may then be NULL (given both,
 *   the keep probability is what is used): where h > 0 the element was kept
 *   and its noise is 1 / keep_prob
 *   dexpert_in [E,R,M]; dwi [E,M,H]; dwo [E,H,N]; everything of `dtype`
 * Four grouped GEMMs on the forward kernels; the weight gradients read both
 * operands as they are (reduction index outermost) where the kernel takes the
 * shape (bf16, kernel dimensions multiples of 8), through transposed copies
 * otherwise.
 */
int mesh_moe_expert_ffn_backward(const void* expert_in, const void* h,
                                 const void* dy, const void* wi,
                                 const void* wo, const void* dh_scale,
                                 float dh_keep_prob,
                                 void* dexpert_in, void* dwi, void* dwo, int E,
                                 int R, int M, int H, int N, int activation,
                                 int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* Bytes of scratch mesh_moe_expert_linear_backward needs. */
size_t mesh_moe_expert_linear_backward_workspace_bytes(int E, int R, int K,
                                                       int N, int dtype);

/*
 * Backward of one expert projection y = a . w (mtf.layers.dense with
 * expert_dims, layers.py:129-208; EinsumOperation.gradient, ops.py:2846-2854):
 *   da = dy . w^T;  dw = a^T . dy
 *   a [E,R,K], dy [E,R,N], w [E,K,N] (the variable's own layout), da [E,R,K]
 *   (NULL: not wanted), dw [E,K,N]; everything of `dtype`
 * With mesh_moe_activation_backward this is what the layer's backward is made
 * of when the experts are not plain ReLU / linear layers (products of several
 * dense layers, other activations: transformer/moe.py:469-475).
 * da_relu_mask [E,R,K] dtype or NULL: da is stored as zero wherever the mask
 * is not positive -- for `a` = relu(...) pass a itself and the ReLU's backward
 * (mtf.relu's gradient, ops.py:1818-1921) is done with the product, on the
 * stores of the GEMM where its kernel can, in a pass of its own otherwise.
 */
int mesh_moe_expert_linear_backward(const void* a, const void* dy,
                                    const void* w, void* da, void* dw,
                                    const void* da_relu_mask, int E, int R,
                                    int K, int N, int dtype, void* workspace,
                                    size_t workspace_bytes, void* stream);

/*
 * out = act(pre) on n elements of `dtype`: the activation of a dense layer
 * (ops.py:1818-1921) as a step of its own, for callers that keep the
 * pre-activation for the backward pass (mesh_moe_expert_linear with that
 * activation gives the same values).
 */
int mesh_moe_activation(const void* pre, void* out, int64_t n, int activation,
                        int dtype, void* stream);

/*
 * dpre = dh * factor * act'(pre) on n elements of `dtype` (float32 arithmetic,
 * one rounding): the gradient of a dense layer's activation from its
 * pre-activation (ops.py:1818-1921), times the other factors of a product of
 * dense layers (factor NULL: none).
 */
int mesh_moe_activation_backward(const void* dh, const void* pre,
                                 const void* factor, void* dpre, int64_t n,
                                 int activation, int dtype, void* stream);

/* Bytes of scratch mesh_moe_gating_backward needs. */
size_t mesh_moe_gating_backward_workspace_bytes(int G, int E);

/*
 * Backward of the gating (transformer/moe.py:1391-1496 for router 0 = top-2,
 * :1207-1306 for router 1 = switch / switch_max, :831-934 for router 2 = ntlb
 * with its top_k and softmax_dtype as in mesh_moe_ntlb_gating; both are
 * ignored otherwise): d(logits) from the
 * gradients of the two combine weights and of the layer's returned loss.
 * With softmax_dtype bfloat16 (ntlb) the probabilities and the candidates are
 * recomputed with the forward's roundings and the float32 derivative of the
 * softmax is evaluated at those probabilities.
 *   logits [G,S,E] float32 (the forward values), importance and
 *   importance_from_slot_gate as in the forward
 *   idx, kept [G,S,2] from the forward; dgate [G,S,2] float32 from
 *   mesh_moe_combine_backward
 *   d_loss [1] float32 ON THE DEVICE: gradient w.r.t. the returned loss
 *   (balancing loss * moe_loss_coef); loss_scale = moe_loss_coef
 *   use_second_place_loss (router 0 only, moe.py:1425-1438) / use_z_loss /
 *   z_loss_coef / num_microbatches as in the forward call
 *   dlogits [G,S,E] float32
 */
int mesh_moe_gating_backward(const float* logits, const void* importance,
                             int importance_dtype,
                             int importance_from_slot_gate, const int32_t* idx,
                             const uint8_t* kept, const float* dgate,
                             const float* d_loss, double loss_scale, int G,
                             int S, int E, int router, int top_k,
                             int softmax_dtype, int use_second_place_loss,
                             int use_z_loss, double z_loss_coef,
                             int num_microbatches,
                             float* dlogits, void* workspace,
                             size_t workspace_bytes, void* stream);

/*
 * Backward of the router projection w.r.t. its kernel
 * (transformer/moe.py:1384-1390): dw_gate[m,e] = sum_t float(x[t,m]) *
 * dlogits[t,e], float32 accumulate, stored in dtype.
 *   x [tokens,M] dtype; dlogits [tokens,E] float32; dw_gate [M,E] dtype
 *   workspace: mesh_moe_router_backward_weights_workspace_bytes(tokens, M, E,
 *   dtype) bytes (M*E float32, or one such plane per chunk of tokens for the
 *   bf16 kernel that sums its chunks in a fixed order)
 */
size_t mesh_moe_router_backward_weights_workspace_bytes(int64_t tokens, int M,
                                                        int E, int dtype);
int mesh_moe_router_backward_weights(const void* x, const float* dlogits,
                                     void* dw_gate, float* workspace,
                                     int64_t tokens, int M, int E, int dtype,
                                     void* stream);

/*
 * Backward of the dispatch einsum (transformer/moe.py:443-447) plus, when
 * dlogits is given, of the router projection w.r.t. the tokens:
 *   dx[g,s,:] = sum over the dispatched choices k of dexpert_in[idx_k,g,pos_k,:]
 *               + dlogits[g,s,:] . w_gate^T
 * float32 accumulate, one rounding.  The dispatch tensor itself carries no
 * gradient (it is a bool cast, moe.py:1510-1511).
 *   dexpert_in [E,G,C,M] dtype; dlogits [G,S,E] float32 or NULL;
 *   w_gate_packed [G / groups_per_router, E, M] dtype (NULL iff dlogits is):
 *   one router per groups_per_router consecutive groups (G for a single
 *   router; the inner level of the hierarchical layer has one per outer
 *   expert, moe.py:743-753); dx [G,S,M] dtype
 *   w_gate [G / groups_per_router, M, E] dtype or NULL: the same router
 *   kernels in their variable layout.  Given them, bf16 calls with
 *   M % 256 == 0, E % 16 == 0, E <= 128 and S % 32 == 0 compute the router's
 *   share on the matrix cores (d(logits) as two bf16 terms; sums in another
 *   order than the other kernels', equal to rounding).
 */
int mesh_moe_dispatch_backward(const void* dexpert_in, const int32_t* idx,
                               const int32_t* pos, const float* gate,
                               const uint8_t* kept, const float* dlogits,
                               const void* w_gate_packed, const void* w_gate,
                               int groups_per_router, void* dx, int G, int S,
                               int E, int C, int M, int dtype, void* stream);

/*
 * The gradient calls on COMPACTED rows, for a layer whose forward pass ran
 * mesh_moe_compact_expert_ffn (routers with one choice per token,
 * transformer/moe.py:1176-1309, :804-940): every tensor with slot rows
 * (expert_in, h, y and their gradients, [E, G*C, .]) holds expert e's occupied
 * slots at rows 0 .. used_e - 1 of its row range, slot (e, g, c) at row
 * row_offsets[e][g] + c, and the four gradient GEMMs skip the rest: the
 * einsum gradients of ops.py:2846-2854 over the occupied slots only.
 * fill [G,E] and row_offsets [E,G] as for mesh_moe_compact_expert_ffn.  Rows
 * from used_e up to the next multiple of 256 are written as zeros by
 * dispatch_compact and combine_backward_compact and stay zero through the
 * GEMMs; rows beyond hold unspecified values that nothing reads.
 *
 * mesh_moe_dispatch_compact: mesh_moe_dispatch into compacted rows
 *   (expert_in [E, G*C, M]; the weight gradient of wi reads it).
 * mesh_moe_combine_backward_compact: mesh_moe_combine_backward with y and dy
 *   in compacted rows.
 * mesh_moe_compact_expert_ffn_backward: mesh_moe_expert_ffn_backward
 *   (relu or linear experts; dh_scale and dh_keep_prob as there); bf16, E <= 1024 and shapes the
 *   256 x 256 kernels take, else MESH_MOE_E_UNSUPPORTED;
 *   ..._workspace_bytes returns 0 for shapes it does not take.
 * mesh_moe_dispatch_backward_compact: mesh_moe_dispatch_backward reading
 *   dexpert_in in compacted rows.
 */
int mesh_moe_dispatch_compact(const void* x, const int32_t* idx,
                              const int32_t* pos, const float* gate,
                              const uint8_t* kept, const int32_t* fill,
                              const int32_t* row_offsets, void* expert_in,
                              int G, int S, int E, int C, int M, int dtype,
                              void* stream);
int mesh_moe_combine_backward_compact(
    const void* dout, const void* y, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* fill,
    const int32_t* row_offsets, void* dy, float* dgate, int G, int S, int E,
    int C, int N, int dtype, void* stream);
size_t mesh_moe_compact_expert_ffn_backward_workspace_bytes(int G, int E, int C,
                                                            int M, int H,
                                                            int N);
int mesh_moe_compact_expert_ffn_backward(
    const void* expert_in, const void* h, const void* dy, const void* wi,
    const void* wo, const void* dh_scale, float dh_keep_prob,
    const int32_t* fill, const int32_t* row_offsets, void* dexpert_in,
    void* dwi, void* dwo, int G, int E, int C, int M, int H, int N,
    int activation, int dtype, void* workspace, size_t workspace_bytes,
    void* stream);
int mesh_moe_dispatch_backward_compact(
    const void* dexpert_in, const int32_t* idx, const int32_t* pos,
    const float* gate, const uint8_t* kept, const int32_t* row_offsets,
    const float* dlogits, const void* w_gate_packed, const void* w_gate,
    int groups_per_router, void* dx, int G, int S, int E, int C, int M,
    int dtype, void* stream);

/*
 * ---------------------------------------------------------------------------
 * The rest of a transformer block around the layer (the LayerStack sublayers
 * and SelfAttention of mesh_tensorflow/transformer/transformer.py and
 * transformer_layers.py).  Dense projections use mesh_moe_expert_linear with
 * E = 1.
 * ---------------------------------------------------------------------------
 */

/*
 * Backward passes of the block's operations.  The reference has no code for
 * them: mtf.gradients differentiates the einsum, reduce and cwise operations
 * these forward kernels fuse (mesh_tensorflow/ops.py:2846-2854 einsum,
 * :1478-1482 gradient hook), so each entry states the derivative it computes.
 * Float32 arithmetic on the stored operands, one rounding to `dtype`.
 *
 * mesh_moe_rms_norm_backward (sublayer_rms_norm, transformer/transformer.py:
 * 493-516): y = x * r * scale with r = rsqrt(mean(x^2) + epsilon);
 *   dx = r * g - x * r^3 * mean(g * x),  g = dy * scale;   dscale = sum_rows dy * x * r.
 * x, dy, dx [rows, M]; scale, dscale [M].
 *
 * mesh_moe_softmax_backward (mtf.softmax, ops.py:5539-5541): from the output w,
 *   dlogits = w * (dw - sum_k dw * w) over the last dim; [rows, L] each.
 *
 * mesh_moe_attention_weights (transformer/attention.py:76-81): the weights
 * softmax(q . k + visibility) the fused forward kernel never stores, recomputed
 * for the backward pass: q, k [B, L, H*D] -> weights [B*H, L, L] in `dtype`
 * (float32 logits and softmax, as in the forward pass).
 */
size_t mesh_moe_rms_norm_backward_workspace_bytes(int64_t rows, int M);
int mesh_moe_rms_norm_backward(const void* x, const void* scale, const void* dy,
                               void* dx, void* dscale, int64_t rows, int M,
                               double epsilon, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream);
int mesh_moe_softmax_backward(const void* weights, const void* dweights,
                              void* dlogits, int64_t rows, int L, int dtype,
                              void* stream);
size_t mesh_moe_attention_weights_workspace_bytes(int B, int L, int H, int D,
                                                  int dtype);
int mesh_moe_attention_weights(const void* q, const void* k, void* weights,
                               int B, int L, int H, int D, int causal,
                               const int32_t* sequence_id,
                               const void* rel_values, const int32_t* rel_bucket,
                               int num_buckets, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream);

/*
 * Dropout whose noise is broadcast over some dimensions of x
 * (mtf.dropout with a noise_shape, mesh_tensorflow/ops.py:5832-5872, as called by
 * sublayer_dropout, transformer/transformer.py:590-599, by dense_relu_dense,
 * layers.py:1176-1178, and on the attention weights, transformer/attention.py:82-84):
 * x and out [outer, mid, inner], uniform / noise_in / noise_out [outer, inner].
 *   out[o, m, i] = x[o, m, i] * noise[o, i]
 *   noise = (uniform < keep_prob) ? 1 / keep_prob : 0   (threshold and quotient
 *           rounded to `dtype`, as scalars of the tensor's type are there)
 * or noise = noise_in (the backward pass: dx = dy * noise).  Exactly one of
 * uniform and noise_in is non-NULL; noise_out may be NULL; out does not overlap x.
 */
int mesh_moe_broadcast_dropout(const void* x, const void* uniform,
                               const void* noise_in, float keep_prob, void* out,
                               void* noise_out, int64_t outer, int64_t mid,
                               int64_t inner, int dtype, void* stream);

/*
 * RMS normalisation (sublayer_rms_norm, transformer/transformer.py:493-516):
 * y = x * rsqrt(mean(square(x)) + epsilon) * scale over the last dim, one
 * rounding to dtype per reference op, float32 accumulation.
 *   x, y [rows,M] dtype; scale [M] dtype
 */
int mesh_moe_rms_norm(const void* x, const void* scale, void* y, int64_t rows,
                      int M, double epsilon, int dtype, void* stream);

/* Bytes of scratch mesh_moe_self_attention needs. */
size_t mesh_moe_self_attention_workspace_bytes(int B, int L, int H, int D,
                                               int dtype, int relative_bias);

/*
 * Multi-head dot-product self-attention after the q/k/v projections
 * (attention.attention with float32_logits, transformer/attention.py:27-88):
 * float32 logits q . k (no scaling: the reference folds 1/sqrt(d_kv) into the
 * query kernel's initialiser, attention.py:436-439), keys after the query
 * masked when `causal` (the autoregressive bias of
 * transformer_layers.py:289-296 via attention.py:830-842), float32 softmax,
 * weights cast to dtype, outputs = weights . v.
 *   q, k, v, out [B,L,H*D] dtype (heads and d_kv combined as the reference's
 *   combine_dims does); any L and D (bf16 shapes whose L or D is not a
 *   multiple of 8 run their two products on a plain tile kernel).
 * bf16 with D = 64 or 128 runs one fused kernel (logits stay on chip, the
 * division by the softmax sum comes after the weights are rounded; no scratch
 * but the bias table below).  Other cases run the three-step form whose logits
 * and weights of all heads live in the workspace (B*H*L*L*(4 + sizeof dtype)
 * bytes).
 * sequence_id [B,L] int32 or NULL: with it a query sees only the keys that
 * carry its own id -- packed sequences and padding (id 0), the visibility
 * bias of SelfAttention.compute_bias, transformer/transformer_layers.py:303-316;
 * mesh_moe_attention_weights and mesh_moe_self_attention_backward take the
 * same argument.
 * rel_values [H,num_buckets] dtype and rel_bucket [2L-1] int32, or both NULL:
 * the relative attention bias of transformer_layers.py:317-352 -- logit (i, j)
 * gets rel_values[h][rel_bucket[j - i + L - 1]], rel_bucket being the bucket of
 * every (memory position - query position) (the caller evaluates
 * _relative_position_bucket, :1000-1042, once per length).  Pass
 * relative_bias = 1 to mesh_moe_self_attention_workspace_bytes; the fused
 * kernel reads the bias from a float32 table [H, 2L-1] it first builds in the
 * workspace.  mesh_moe_attention_weights takes the same arguments.
 * lse [B*H,L] float32 or NULL: where the fused kernel runs
 * (mesh_moe_self_attention_backward_workspace_bytes > 0 for the shape) it also
 * writes the logarithm of every query's softmax denominator, which
 * mesh_moe_self_attention_backward takes back; MESH_MOE_E_UNSUPPORTED where
 * the three-step form runs.
 */
int mesh_moe_self_attention(const void* q, const void* k, const void* v,
                            void* out, int B, int L, int H, int D, int causal,
                            const int32_t* sequence_id, const void* rel_values,
                            const int32_t* rel_bucket, int num_buckets,
                            float* lse, int dtype, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * Gradient of the relative attention bias values (the gradient of the
 * mtf.gather at transformer/transformer_layers.py:351):
 * dvalues[h][bucket] = sum over the batch and the (query i, key j) pairs with
 * rel_bucket[j - i + L - 1] == bucket of dlogits[b*H + h][i][j].
 *   dlogits [B*H,L,L] dtype (what mesh_moe_softmax_backward writes);
 *   dvalues [H,num_buckets] dtype; workspace H*num_buckets floats.
 * Float32 atomics: the order of the sum is not fixed.
 */
int mesh_moe_relative_bias_backward(const void* dlogits,
                                    const int32_t* rel_bucket, void* dvalues,
                                    float* workspace, int B, int L, int H,
                                    int num_buckets, int dtype, void* stream);

/* Bytes of scratch mesh_moe_self_attention_backward needs; 0 for shapes it does
 * not take. */
size_t mesh_moe_self_attention_backward_workspace_bytes(int B, int L, int H,
                                                        int D, int dtype,
                                                        int relative_bias);

/*
 * Backward of mesh_moe_self_attention in fused kernels: what mtf.gradients
 * (mesh_tensorflow/ops.py:5254-5291) assembles from the gradients of the two
 * einsums and the softmax of attention.attention
 * (transformer/attention.py:76-87).  With W = softmax(q . k) cast to dtype:
 *   dW = dout . v^T,  delta = sum_k dW W,  dS = W (dW - delta) cast to dtype,
 *   dv = W^T . dout,  dq = dS . k,  dk = dS^T . q.
 *   q, k, v, dout, dq, dk, dv [B,L,H*D] dtype.
 * bf16 with D = 64 or 128 and L a multiple of 8 only (MESH_MOE_E_UNSUPPORTED
 * otherwise: compose mesh_moe_attention_weights, mesh_moe_softmax_backward and
 * mesh_moe_expert_linear_backward instead).  Nothing of size L x L reaches
 * memory; the workspace holds two float32 [B*H, L] vectors.  Four launches:
 * one pass in the forward kernel's shape for the softmax denominators and
 * delta, then one kernel per output, each recomputing W per tile, so that
 * every output element is summed by one wavefront in a fixed order (no
 * atomics; the same bits on every run).  dW is not rounded to dtype before
 * the subtraction and delta comes from sum_d dout out in float32 -- fewer
 * roundings than the reference's chain of ops, inside its tolerance.
 * rel_values, rel_bucket, num_buckets as for mesh_moe_self_attention, with
 * dvalues [H,num_buckets] dtype (all NULL / 0: no bias): W is recomputed with
 * the bias and dvalues receives the gradient of rel_values (the gradient of
 * the mtf.gather at transformer_layers.py:351): the dq kernel sums its dS
 * (float32, before the cast) along the diagonals into a float32 table
 * [H, 2L-1] with atomics -- the order of that sum is not fixed -- and a last
 * small kernel adds up each bucket's distances.
 * out [B,L,H*D] dtype and lse [B*H,L] float32 (both or neither): what
 * mesh_moe_self_attention wrote for the same arguments.  With them the first
 * of the four launches is replaced by a small one (delta = sum_d dout out from
 * the rounded outputs); without them the denominators are recomputed.
 */
int mesh_moe_self_attention_backward(const void* q, const void* k, const void* v,
                                     const void* dout, void* dq, void* dk,
                                     void* dv, int B, int L, int H, int D,
                                     int causal, const int32_t* sequence_id,
                                     const void* rel_values,
                                     const int32_t* rel_bucket, int num_buckets,
                                     void* dvalues, const void* out,
                                     const float* lse, int dtype,
                                     void* workspace, size_t workspace_bytes,
                                     void* stream);

/*
 * One decoding step of self-attention: SelfAttention.call in "incremental"
 * mode (transformer/transformer_layers.py:231-254) with the visibility of
 * :289-296.  The step's key and value replace row position[b] of the recurrent
 * states (the reference's k = old_k * (1 - one_hot) + k * one_hot, here in
 * place), the query sees memory positions m <= position[b]; float32 logits and
 * softmax, weights cast to dtype, out = weights . v.
 *   q, k_new, v_new, out [B,H*D] dtype; k_cache, v_cache [B,Lm,H*D] dtype,
 *   updated in place; position [B] int32 on the device, clamped to [0, Lm).
 * One block per (head, batch entry), the caches read once.  Lm up to ~36000
 * (the logits of a row live in LDS).
 * rel_values [H,num_buckets] dtype and rel_bucket [2*Lm-1] int32, or both NULL:
 * the relative attention bias of the step (compute_bias with context.position,
 * transformer_layers.py:317-352): the logit of memory position m gets
 * rel_values[h][rel_bucket[m - position[b] + Lm - 1]].
 */
int mesh_moe_attention_decode(const void* q, const void* k_new, const void* v_new,
                              void* k_cache, void* v_cache,
                              const int32_t* position, void* out, int B, int Lm,
                              int H, int D, const void* rel_values,
                              const int32_t* rel_bucket, int num_buckets,
                              int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* MESH_MOE_H_ */
