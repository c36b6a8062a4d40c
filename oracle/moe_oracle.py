"""CPU restatement of Mesh TensorFlow's top-2 Mixture-of-Experts forward path.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Every function restates, in NumPy float32 arithmetic with one rounding per
reference op, what the reference's single-device lowering computes.  The
reference builds the layer from ~100 separately lowered primitives; each line
below that performs arithmetic corresponds to one of those primitives, so the
rounding points are the reference's.

What pins each function (the reference holds no test or golden vector of its
MoE file, and its TensorFlow dependency cannot run here):

  split_into_groups, expert_capacity  brute force over the defining
                                      constraints + the five config capacities
  softmax                             float64 scipy softmax, row-sum invariant
  top_1 / top-2 selection             stable argsort brute force, exact ties
  capacity positions / drops          sequential integer loop
                                      (routing_sequential) + a hand-worked case
  combine / dispatch tensors          rebuilt from (idx, pos, gate, kept)
  dispatch / combine einsums          gather/scatter form vs np.einsum
  expert FFN                          float64 matmul
  aux loss                            balanced-routing closed form (= 1.0)
  switch_gating                       sequential integer loop, raw-probability
                                      gate vs float64 softmax, closed forms for
                                      the loss (balanced: = fraction of tokens
                                      with importance 1) and the z-loss
                                      (constant logits c: (c + log E)^2 / mb)
  switch_max_gating                   repeated arg-max selection (the k < 5
                                      lowering of mtf.top_k) vs the stable
                                      sort, per-expert brute force, equality
                                      with switch_gating when nothing overflows
  ntlb_gating                         walk over (pass, token) with one
                                      counter per expert, a hand-worked case
                                      (4 tokens, 3 experts, capacity 1),
                                      k = 1 equals switch_gating, closed-form
                                      loss (uniform router: 1.0 for any k),
                                      dense tensors vs record
  softmax_bf16 (ntlb with bfloat16    two rows worked by hand, the op chain in
  activations, moe.py:825-836)        Python floats with a frexp-based
                                      rounding, one-hot rows (every op exact)
                                      equal the float32 chain, a by-hand tie
                                      case through the router; UNPINNED: the
                                      float32 accumulation order inside
                                      TensorFlow's bfloat16 reduce_sum (index
                                      order here; rounded once either way)
  expert_selection_gating             per-expert stable sort brute force,
                                      weights of a token sum to sum(p)/count,
                                      closed-form loss (uniform logits: 1.0),
                                      dense tensors vs slot record
  router_summaries                    closed forms (uniform logits: entropy
                                      log E, expert_gate 1 / E, all choices on
                                      expert 0, z-loss (log E)^2 / mb; one-hot
                                      rows: entropy 0, gate 1), a per-token
                                      float64 loop, fraction_routed against the
                                      capacity (S tokens on one expert:
                                      C / S), group_token sums to G E C E C
  perturb_gate_inputs                 closed forms (eps = 0 and eval change
                                      nothing, all-kept dropout scales the
                                      logits by 1 / keep_prob), the experts
                                      see the unperturbed tokens; backward by
                                      central differences with the multiplier
                                      held fixed
  expert_hidden (products of dense    independent float64 evaluation per
  layers), hidden_dropout_noise       activation pair, factors commute, a zero
                                      linear factor zeroes the output; the
                                      noise against torch's arithmetic in the
                                      tensor's dtype, strict threshold, keep
                                      0.5 with everything kept = twice the
                                      plain layer; backward through the
                                      dropout by central differences
  gating_backward,                    central differences of an independent
  moe_layer_v1_backward               float64 forward with the routing held
                                      fixed (tests/test_oracle.py), every
                                      router (expert selection included), the
                                      second-place loss, the noise policies,
                                      the hidden dropout, other activations
                                      and products of dense layers
  v2                                  x=1 outer expert reduces to v1

PARITY UNPINNED against TensorFlow itself (only running the reference could
pin these): near-tie behaviour of argmax after TF's exp/log, the accumulation
order of TF's bf16 einsum, and the random streams (the "random" second-place
policy, the router input noise, the hidden dropout): the uniform numbers are
explicit inputs here.

Citations are to files under the reference tree (mesh_tensorflow/...).
"""

import numpy as np

F32 = np.float32


# ----------------------------------------------------------------------------
# dtype helpers
# ----------------------------------------------------------------------------
def round_bf16(a):
  """float32 -> bfloat16 (round to nearest even) -> float32.

  Stands in for tf.cast(x, tf.bfloat16) (ops.py:1945-1951).
  """
  shape = np.shape(a)
  a = np.ascontiguousarray(a, dtype=F32).reshape(-1)
  u = a.view(np.uint32)
  nan = np.isnan(a)
  rounded = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))))
  rounded = rounded & np.uint32(0xFFFF0000)
  out = rounded.view(F32).copy()
  if nan.any():
    out[nan] = np.nan
  return out.reshape(shape)


def cast_act(a, act_dtype):
  """tf.cast to the activation dtype ("float32" or "bfloat16")."""
  if act_dtype == "bfloat16":
    return round_bf16(a)
  if act_dtype == "float32":
    return np.asarray(a, dtype=F32)
  raise ValueError("unsupported activation dtype %r" % (act_dtype,))


# ----------------------------------------------------------------------------
# host integer logic
# ----------------------------------------------------------------------------
def split_into_groups(n, max_group_size, mesh_dim_size):
  """transformer/moe.py:1549-1582."""
  if n % mesh_dim_size != 0:
    raise ValueError(
        "n=%d is not a multiple of mesh_dim_size=%d" % (n, mesh_dim_size))
  num_groups = max(1, n // max_group_size)
  while num_groups % mesh_dim_size != 0 or n % num_groups != 0:
    num_groups += 1
  return num_groups, n // num_groups


def expert_capacity(group_size, capacity_factor, num_experts,
                    min_expert_capacity):
  """transformer/moe.py:368-371 (v2: :671-672, :686-689)."""
  c = min(group_size, int((group_size * capacity_factor) / num_experts))
  return max(c, min_expert_capacity)


# ----------------------------------------------------------------------------
# mtf primitives, restated
# ----------------------------------------------------------------------------
def seq_sum(x, axis=-1):
  """Sequential float32 sum in index order (the order tf.reduce_sum uses is
  Eigen's and is not specified; this is the order the HIP kernels use)."""
  x = np.asarray(x, dtype=F32)
  return np.add.accumulate(x, axis=axis, dtype=F32).take(-1, axis=axis)


def softmax(x):
  """mtf.softmax over the last axis: exp(x - logsumexp(x)).

  ops.py:5539-5541 -> log_softmax :5523-5536 -> reduce_logsumexp :5493-5520.
  Subtraction is add(x, negative(y)) (ops.py:5116-5132).
  """
  x = np.asarray(x, dtype=F32)
  m = x.max(axis=-1, keepdims=True)                      # reduce_max
  t = x + (-m)                                           # x -= max_logit
  u = np.exp(t).astype(F32)                              # exp
  s = seq_sum(u, axis=-1)[..., None]                     # reduce_sum
  lse = np.log(s).astype(F32) + m                        # log(...) + max_logit
  return np.exp(x + (-lse)).astype(F32)                  # exp(log_softmax)


def softmax_bf16(x):
  """mtf.softmax over the last axis of a bfloat16 tensor, as float32 values
  that are all bfloat16-representable.

  The same op chain as softmax() (ops.py:5493-5541), but every op of it is a
  TensorFlow op of its own on a bfloat16 tensor and so rounds its result to
  bfloat16: negative and reduce_max are exact; add, exp, log round once (Eigen
  evaluates a bfloat16 exp / log in float32 and rounds the result).
  tf.reduce_sum of a bfloat16 tensor accumulates in float32 and rounds once
  (TensorFlow's sum reducer casts bfloat16 to float, reduction_ops.h); the
  float32 accumulation order is Eigen's and unspecified -- here: index order,
  which after the rounding to bfloat16 almost never matters.
  _ntlb_gating is the one router that runs its softmax in the activation dtype
  (moe.py:825-836: dense -> softmax -> to_float).
  """
  x = round_bf16(x)
  m = x.max(axis=-1, keepdims=True)                      # reduce_max
  t = round_bf16(x + (-m))                               # x -= max_logit
  u = round_bf16(np.exp(t).astype(F32))                  # exp
  s = round_bf16(seq_sum(u, axis=-1))[..., None]         # reduce_sum
  lse = round_bf16(round_bf16(np.log(s).astype(F32)) + m)  # log(...) + max
  return round_bf16(np.exp(round_bf16(x + (-lse))).astype(F32))


def router_softmax(logits, gating, act_dtype):
  """The router's probabilities from float32-accumulated logits.  top_2,
  switch, switch_max and expert_selection cast the tokens to float32 before
  the projection (moe.py:1384, :1201, :1080); _ntlb_gating does not: its
  projection's result and its softmax have the activation dtype and only the
  probabilities are cast to float32 (moe.py:825-836)."""
  if gating == "ntlb" and act_dtype == "bfloat16":
    return softmax_bf16(logits)
  return softmax(logits)


def top_1(x):
  """mtf.top_1 over the last axis: (reduce_max, int32 first argmax).

  ops.py:5018-5033 -> TopKOperation k=1 branch ops.py:4937-4940.
  """
  return x.max(axis=-1), np.argmax(x, axis=-1).astype(np.int32)


def one_hot(idx, depth):
  """tf.one_hot semantics: an out-of-range index gives an all-zero row
  (ops.py:3830-3851)."""
  idx = np.asarray(idx)
  return (idx[..., None] == np.arange(depth, dtype=idx.dtype)).astype(F32)


def cumsum_exclusive(x, dense=False):
  """mtf.cumsum(x, group_size_dim, exclusive=True) for x of shape [..., S, E].

  ops.py:2761-2781 implements it as an einsum with an S x S triangular 0/1
  matrix.  With dense=True that matmul is performed literally (used for the CPU
  baseline timing and on tiny cases); otherwise np.cumsum is used, which gives
  identical values because every partial sum is an integer below 2**24.
  """
  x = np.asarray(x, dtype=F32)
  s = x.shape[-2]
  if dense:
    r = np.arange(s, dtype=F32)
    tri = (r[:, None] < r[None, :]).astype(F32)          # [s, s'] = s < s'
    return np.einsum("...se,st->...te", x, tri).astype(F32)
  return (np.cumsum(x, axis=-2, dtype=F32) - x).astype(F32)


# ----------------------------------------------------------------------------
# _top_2_gating  (transformer/moe.py:1312-1513)
# ----------------------------------------------------------------------------
def top_2_gating(logits, capacity, importance=None, policy="all",
                 threshold=0.2, use_second_place_loss=False,
                 num_microbatches=None, act_dtype="float32",
                 second_uniform=None, dense=False):
  """Everything in _top_2_gating after the router projection.

  Args:
    logits: float32 [G, S, E] router logits (output of the `dense` at
      moe.py:1386-1390; leading dims may be flattened into G).
    capacity: int, expert_capacity_dim.size.
    importance: optional float [G, S].
    policy, threshold: moe_second_policy_* / moe_second_threshold_*.
    second_uniform: U(0,1) samples [G, S] for policy "random" (the reference
      draws them with mtf.random_uniform, moe.py:1464).
    dense: build the dense [G,S,E,C] tensors and use the S x S cumsum matmul.

  Returns a dict with
    combine, dispatch: [G,S,E,C] in the activation dtype (only if dense),
    loss: float32 scalar cast to the activation dtype (moe.py:1508),
    index_1/2 int32 [G,S], pos_1/2 int32 [G,S] (raw, meaningful where kept),
    kept_1/2 bool [G,S] (mask_k_flat), gate_1/2 float32 [G,S] (after the
    multiplication by mask_k_flat, before the activation-dtype cast),
    fill int32 [G,E] occupied slots per expert.
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  cap_f = F32(float(capacity))

  raw_gates = softmax(logits)                                    # :1391
  gate_1, index_1 = top_1(raw_gates)                             # :1397
  mask_1 = one_hot(index_1, e_)                                  # :1399
  density_1_proxy = raw_gates                                    # :1400
  if importance is not None:
    importance = np.asarray(importance, dtype=F32)
    is_one = (importance == F32(1.0)).astype(F32)                # :1402-1404
    mask_1 = mask_1 * is_one[..., None]
    gate_1 = gate_1 * is_one
    density_1_proxy = density_1_proxy * is_one[..., None]
  gates_without_top_1 = raw_gates * (F32(1.0) + (-mask_1))       # :1405
  gate_2, index_2 = top_1(gates_without_top_1)                   # :1407
  mask_2 = one_hot(index_2, e_)                                  # :1409
  if importance is not None:
    mask_2 = mask_2 * (importance > F32(0.0)).astype(F32)[..., None]  # :1411

  denom = (gate_1 + gate_2) + F32(1e-9)                          # :1413
  recip = (F32(1.0) / denom).astype(F32)                         # reciprocal
  gate_1 = gate_1 * recip                                        # :1414
  gate_2 = gate_2 * recip                                        # :1415

  # balancing loss (:1420-1442); reduce_mean = reduce_sum * (out/in), the
  # Python quotient becoming a float32 scalar (ops.py:4804-4808).
  inv_s = F32(1.0 / s_)
  density_1 = seq_sum(mask_1, axis=-2) * inv_s                   # [G,E]
  density_1_proxy = seq_sum(density_1_proxy, axis=-2) * inv_s    # [G,E]
  prod = density_1_proxy * density_1
  loss = seq_sum(prod.reshape(-1)) * F32(1.0 / prod.size)
  loss = loss * F32(float(e_ * e_))
  if use_second_place_loss:                                      # :1426-1438
    density_2 = seq_sum(mask_2, axis=-2) * inv_s
    qsum = seq_sum(gates_without_top_1, axis=-1) + F32(1e-9)
    normalized = gates_without_top_1 * (F32(1.0) / qsum).astype(F32)[..., None]
    density_2_proxy = seq_sum(normalized, axis=-2) * inv_s
    prod2 = density_2_proxy * density_2
    loss_2 = seq_sum(prod2.reshape(-1)) * F32(1.0 / prod2.size)
    loss_2 = loss_2 * F32(float(e_ * e_))
    loss = loss + loss_2 * F32(0.5)
  if num_microbatches and num_microbatches > 1:                  # :1439-1442
    loss = loss * F32(1.0 / num_microbatches)

  if policy == "all":                                            # :1452-1467
    pass
  elif policy == "none":
    mask_2 = np.zeros_like(mask_2)
  elif policy == "threshold":
    mask_2 = mask_2 * (gate_2 > F32(threshold)).astype(F32)[..., None]
  elif policy == "random":
    if second_uniform is None:
      raise ValueError("policy 'random' needs second_uniform samples")
    u = np.asarray(second_uniform, dtype=F32)
    lim = gate_2 * F32(1.0 / max(threshold, 1e-9))
    mask_2 = mask_2 * (u < lim).astype(F32)[..., None]
  else:
    raise ValueError("Unknown policy %s" % policy)

  # capacity assignment (:1472-1496)
  position_in_expert_1 = cumsum_exclusive(mask_1, dense) * mask_1
  mask_1 = mask_1 * (position_in_expert_1 < cap_f).astype(F32)
  mask_1_count = seq_sum(mask_1, axis=-2)                        # [G,E]
  mask_1_flat = seq_sum(mask_1, axis=-1)                         # [G,S]
  position_in_expert_1 = seq_sum(position_in_expert_1, axis=-1)
  gate_1 = gate_1 * mask_1_flat

  position_in_expert_2 = (
      cumsum_exclusive(mask_2, dense) + mask_1_count[:, None, :])
  position_in_expert_2 = position_in_expert_2 * mask_2
  mask_2 = mask_2 * (position_in_expert_2 < cap_f).astype(F32)
  mask_2_flat = seq_sum(mask_2, axis=-1)
  gate_2 = gate_2 * mask_2_flat
  position_in_expert_2 = seq_sum(position_in_expert_2, axis=-1)

  pos_1 = position_in_expert_1.astype(np.int32)                  # to_int32
  pos_2 = position_in_expert_2.astype(np.int32)
  out = dict(
      index_1=index_1, index_2=index_2, pos_1=pos_1, pos_2=pos_2,
      kept_1=mask_1_flat > 0, kept_2=mask_2_flat > 0,
      gate_1=gate_1, gate_2=gate_2,
      fill=(mask_1_count + seq_sum(mask_2, axis=-2)).astype(np.int32),
      loss=cast_act(loss, act_dtype)[()])                        # :1508
  if dense:
    combine = (                                                  # :1499-1505
        (gate_1 * mask_1_flat)[..., None, None]
        * one_hot(index_1, e_)[..., None]
        * one_hot(pos_1, capacity)[..., None, :]
        + (gate_2 * mask_2_flat)[..., None, None]
        * one_hot(index_2, e_)[..., None]
        * one_hot(pos_2, capacity)[..., None, :])
    combine = cast_act(combine, act_dtype)                       # :1507
    out["combine"] = combine
    out["dispatch"] = (combine != 0).astype(F32)                 # :1510-1511
  return out


# ----------------------------------------------------------------------------
# _switch_gating  (transformer/moe.py:1176-1309)
# ----------------------------------------------------------------------------
def sample_choice_logits(logits, temperature, uniform):
  """mtf.sample_with_temperature before its argmax (ops.py:5070-5086): logits +
  g * temperature with Gumbel noise g = -log(-log(u)), u in [1e-9, 1).
  `uniform` stands in for random_uniform's U[0, 1) draw."""
  logits = np.asarray(logits, F32)
  if temperature == 0.0:
    return logits
  tiny = F32(1e-9)
  u = tiny + np.asarray(uniform, F32) * (F32(1.0) - tiny)
  g = -np.log(-np.log(u).astype(F32)).astype(F32)
  return (logits + g * F32(temperature)).astype(F32)


def switch_gating(logits, capacity, importance=None, train=False, z_loss=None,
                  num_microbatches=None, act_dtype="float32", dense=False,
                  choice_logits=None):
  """Everything in _switch_gating after the router projection, for the
  deterministic policies ("argmax"; "input_dropout" / "input_jitter" when not
  training, where they change nothing, moe.py:1192-1199).

  Same arguments and result dict as top_2_gating; the second-choice entries
  are all "not kept" so that dispatch_gather / combine_gather apply unchanged.
  The gate is the raw softmax probability of the chosen expert (no
  normalisation).  z_loss (hparams.moe_z_loss) is added only when training
  (moe.py:1253); the reference then needs `importance` and `num_microbatches`
  (it evaluates equal(importance, 1.0) and denom * num_microbatches
  unconditionally, moe.py:1260-1264) and so does this function.
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  cap_f = F32(float(capacity))

  raw_gates = softmax(logits)                                    # :1207
  if choice_logits is None:
    expert_gate, expert_index = top_1(raw_gates)                 # :1210
  else:    # policy "sample" (:1213-1216): argmax elsewhere, gate gathered
    expert_index = np.argmax(np.asarray(choice_logits, F32), -1).astype(np.int32)
    expert_gate = np.take_along_axis(raw_gates, expert_index[..., None],
                                     -1)[..., 0]
  expert_mask = one_hot(expert_index, e_)                        # :1221

  # load balancing loss (:1224-1238).  density_1 is taken BEFORE the
  # importance mask; density_1_proxy [G,E] times (importance == 1) [G,S]
  # broadcasts to [G,E,S] and the mean runs over all three dims.
  inv_s = F32(1.0 / s_)
  density_1 = seq_sum(expert_mask, axis=-2) * inv_s              # [G,E]
  density_1_proxy = seq_sum(raw_gates, axis=-2) * inv_s          # [G,E]
  is_one = None
  if importance is not None:
    importance = np.asarray(importance, dtype=F32)
    is_one = (importance == F32(1.0)).astype(F32)                # [G,S]
    expert_mask = expert_mask * is_one[..., None]                # :1227
    expert_gate = expert_gate * is_one                           # :1228
    density_1_proxy = density_1_proxy[:, :, None] * is_one[:, None, :]
    prod = density_1_proxy * density_1[:, :, None]               # [G,E,S]
    # G*E*S terms: tf.reduce_sum's order is Eigen's tree, whose error does not
    # grow with the length as a sequential float32 sum's would; a float64
    # accumulation rounded once stands in for it
    total = F32(prod.sum(dtype=np.float64))
  else:
    prod = density_1_proxy * density_1
    total = seq_sum(prod.reshape(-1))
  loss = total * F32(1.0 / prod.size)                            # reduce_mean
  loss = loss * F32(float(e_ * e_))
  if num_microbatches and num_microbatches > 1:                  # :1235-1238
    loss = loss * F32(1.0 / num_microbatches)

  if train and z_loss is not None:                               # :1253-1266
    if is_one is None or not num_microbatches:
      raise ValueError("z_loss needs importance and num_microbatches "
                       "(moe.py:1260-1264)")
    m = logits.max(axis=-1, keepdims=True)                       # :5510-5520
    log_z = np.log(seq_sum(np.exp(logits + (-m)).astype(F32), axis=-1)
                   ).astype(F32) + m[..., 0]
    z = (log_z * log_z) * is_one                                 # square, mask
    denom = seq_sum(is_one.reshape(-1))
    z = seq_sum(z.reshape(-1)) / (denom * F32(num_microbatches))
    loss = loss + F32(z_loss) * z                                # :1266

  # capacity assignment (:1268-1291)
  position_in_expert = cumsum_exclusive(expert_mask, dense) * expert_mask
  expert_mask = expert_mask * (position_in_expert < cap_f).astype(F32)
  expert_mask_flat = seq_sum(expert_mask, axis=-1)               # [G,S]
  expert_gate = expert_gate * expert_mask_flat                   # :1291

  pos_full = position_in_expert.astype(np.int32)                 # [G,S,E]
  pos_1 = np.take_along_axis(pos_full, expert_index[..., None], -1)[..., 0]
  zeros_i = np.zeros_like(expert_index)
  out = dict(
      index_1=expert_index, index_2=zeros_i, pos_1=pos_1, pos_2=zeros_i,
      kept_1=expert_mask_flat > 0, kept_2=np.zeros(expert_index.shape, bool),
      gate_1=expert_gate, gate_2=np.zeros_like(expert_gate),
      fill=seq_sum(expert_mask, axis=-2).astype(np.int32),
      loss=cast_act(loss, act_dtype)[()])                        # :1304
  if dense:
    # one_hot(to_int32(position_in_expert)) is taken per expert ([G,S,E] ->
    # [G,S,E,C]); non-chosen experts have position 0 but a zero one_hot(index)
    combine = (                                                  # :1293-1299
        (expert_gate * expert_mask_flat)[..., None, None]
        * one_hot(expert_index, e_)[..., None]
        * one_hot(pos_full, capacity))
    combine = cast_act(combine, act_dtype)                       # :1302
    out["combine"] = combine
    out["dispatch"] = (combine != 0).astype(F32)                 # :1305-1306
  return out


# ----------------------------------------------------------------------------
# _switch_max_gating  (transformer/moe.py:943-1054)
# ----------------------------------------------------------------------------
def top_k_lowest_index_first(x, k, axis):
  """tf.math.top_k along `axis` as mtf.top_k lowers it (ops.py:4934-4942; for
  1 < k < 5 mtf uses repeated top_1 with the taken entries pushed to -1e9,
  ops.py:4988-5017, which selects the same entries): the k largest values in
  descending order, equal values in ascending index order (the documented
  tie rule of tf.math.top_k).  Returns (values, indices) with k last."""
  x = np.moveaxis(np.asarray(x), axis, -1)
  order = np.argsort(-x, axis=-1, kind="stable")[..., :k].astype(np.int32)
  return np.take_along_axis(x, order, -1), order


def switch_max_gating(logits, capacity, importance=None,
                      num_microbatches=None, act_dtype="float32", dense=False,
                      choice_logits=None):
  """Everything in _switch_max_gating after the router projection, for the
  deterministic policies (as switch_gating).

  Choice, gate and loss are those of _switch_gating (no z-loss here); the
  slots differ: expert e keeps, per group, the `capacity` tokens that chose it
  with the LARGEST gate, slot c holding the (c+1)-th largest
  (top_k over the group dim of expert_mask * expert_gate, moe.py:1033-1039).
  A slot whose selected value is 0 (fewer choosers than slots) combines with
  weight 0 and is therefore not dispatched.  Same result dict as
  switch_gating; pos_1 is the slot, meaningful where kept_1.
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  raw_gates = softmax(logits)                                    # :976
  if choice_logits is None:
    expert_gate, expert_index = top_1(raw_gates)                 # :979
  else:                                                          # :982-985
    expert_index = np.argmax(np.asarray(choice_logits, F32), -1).astype(np.int32)
    expert_gate = np.take_along_axis(raw_gates, expert_index[..., None],
                                     -1)[..., 0]
  expert_mask = one_hot(expert_index, e_)                        # :990
  inv_s = F32(1.0 / s_)
  density_1 = seq_sum(expert_mask, axis=-2) * inv_s              # :994
  density_1_proxy = seq_sum(raw_gates, axis=-2) * inv_s          # :995
  if importance is not None:                                     # :996-1000
    importance = np.asarray(importance, dtype=F32)
    is_one = (importance == F32(1.0)).astype(F32)
    expert_mask = expert_mask * is_one[..., None]
    expert_gate = expert_gate * is_one
    density_1_proxy = density_1_proxy[:, :, None] * is_one[:, None, :]
    prod = density_1_proxy * density_1[:, :, None]
    total = F32(prod.sum(dtype=np.float64))    # see switch_gating
  else:
    prod = density_1_proxy * density_1
    total = seq_sum(prod.reshape(-1))
  loss = total * F32(1.0 / prod.size)
  loss = loss * F32(float(e_ * e_))                              # :1001-1003
  if num_microbatches and num_microbatches > 1:
    loss = loss * F32(1.0 / num_microbatches)

  expert_masked_probs = expert_mask * expert_gate[..., None]     # :1033 [G,S,E]
  probs, tokens = top_k_lowest_index_first(expert_masked_probs, capacity, 1)
  # probs, tokens: [G, E, C]
  kept = np.zeros((g_, s_), bool)
  pos_1 = np.zeros((g_, s_), np.int32)
  gate_1 = np.zeros((g_, s_), F32)
  fill = np.zeros((g_, e_), np.int32)
  for g in range(g_):
    for e in range(e_):
      for c in range(capacity):
        if probs[g, e, c] > 0:
          t = tokens[g, e, c]
          kept[g, t], pos_1[g, t], gate_1[g, t] = True, c, probs[g, e, c]
          fill[g, e] += 1
  zeros_i = np.zeros_like(expert_index)
  out = dict(
      index_1=expert_index, index_2=zeros_i, pos_1=pos_1, pos_2=zeros_i,
      kept_1=kept, kept_2=np.zeros((g_, s_), bool),
      gate_1=gate_1, gate_2=np.zeros((g_, s_), F32), fill=fill,
      loss=cast_act(loss, act_dtype)[()])                        # :1049
  if dense:
    dispatch = one_hot(tokens, s_)                               # [G,E,C,S]
    combine = dispatch * probs[..., None]                        # :1038-1039
    combine = cast_act(combine.transpose(0, 3, 1, 2), act_dtype)  # [G,S,E,C]
    out["combine"] = combine
    out["dispatch"] = (combine != 0).astype(F32)                 # :1050-1051
  return out


# ----------------------------------------------------------------------------
# _ntlb_gating  (transformer/moe.py:804-940)
# ----------------------------------------------------------------------------
def ntlb_gating(logits, capacity, top_k, importance=None,
                num_microbatches=None, act_dtype="float32", dense=False):
  """Everything in _ntlb_gating ("no token left behind") after the router
  projection, for the deterministic policies (as switch_gating).

  Every token names its `top_k` best experts (mtf.top_k, moe.py:839-842).
  Pass i offers the still unrouted tokens to their i-th expert in token
  order; an expert takes them while its running total, carried over from the
  earlier passes, stays within `capacity` (moe.py:905-934).  A token is routed
  at most once; its gate is the raw softmax probability of the expert that
  took it.  Same result dict as switch_gating, plus `taken_in_pass` [G,S] (which of
  its choices took the token, -1 if none) and `topk_index` [G,S,k].
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  k_ = int(top_k)
  if not 1 <= k_ <= e_:
    raise ValueError("moe_ntlb_top_k=%d with %d experts" % (k_, e_))
  raw_gates = router_softmax(logits, "ntlb", act_dtype)          # :831-835
  expert_gate, expert_index = top_k_lowest_index_first(raw_gates, k_, -1)
  expert_mask = one_hot(expert_index, e_)                        # [G,S,k,E]

  # load balancing loss (:845-861): density_1 [G,k,E] before the importance
  # mask; the proxy [G,E] times (importance == 1) [G,S] broadcasts, and the
  # mean runs over every dim of the product
  inv_s = F32(1.0 / s_)
  density_1 = seq_sum(expert_mask, axis=1) * inv_s               # [G,k,E]
  density_1_proxy = seq_sum(raw_gates, axis=-2) * inv_s          # [G,E]
  if importance is not None:
    importance = np.asarray(importance, dtype=F32)
    is_one = (importance == F32(1.0)).astype(F32)                # [G,S]
    expert_mask = expert_mask * is_one[..., None, None]          # :850
    expert_gate = expert_gate * is_one[..., None]                # :851
    proxy = density_1_proxy[:, :, None] * is_one[:, None, :]     # [G,E,S]
    prod = proxy[:, None, :, :] * density_1[..., None]           # [G,k,E,S]
    total = F32(prod.sum(dtype=np.float64))    # see switch_gating
  else:
    prod = density_1_proxy[:, None, :] * density_1               # [G,k,E]
    total = seq_sum(prod.reshape(-1))
  loss = total * F32(1.0 / prod.size)
  loss = loss * F32(float(e_ * e_))                              # :854-856
  if num_microbatches and num_microbatches > 1:                  # :857-860
    loss = loss * F32(1.0 / num_microbatches)

  cap_f = F32(float(capacity))
  cum_tokens = np.zeros((g_, e_), F32)                           # :897-898
  left = np.ones((g_, s_), F32)                                  # :899-900
  index_1 = expert_index[..., 0].copy()
  pos_1 = np.zeros((g_, s_), np.int32)
  gate_1 = np.zeros((g_, s_), F32)
  kept_1 = np.zeros((g_, s_), bool)
  rnd = np.full((g_, s_), -1, np.int32)
  combine = np.zeros((g_, s_, e_, capacity), F32) if dense else None
  for i in range(k_):                                            # :903-934
    mask_i = expert_mask[:, :, i, :] * left[..., None]           # [G,S,E]
    cumulative = cum_tokens[:, None, :] + np.cumsum(mask_i, axis=1, dtype=F32)
    within = (cumulative <= cap_f).astype(F32)                   # :913-914
    out_i = mask_i * within
    cum_tokens = cum_tokens + seq_sum(out_i, axis=1)
    out_flat = seq_sum(out_i, axis=-1)                           # [G,S]
    left = left + (-out_flat)
    position = cumulative - F32(1.0)                             # [G,S,E]
    took = out_flat > 0
    idx_i = expert_index[:, :, i]
    pos_i = np.take_along_axis(position, idx_i[..., None], -1)[..., 0]
    index_1[took] = idx_i[took]
    pos_1[took] = pos_i[took].astype(np.int32)
    gate_1[took] = expert_gate[:, :, i][took]
    kept_1 |= took
    rnd[took] = i
    if dense:
      combine = combine + (                                      # :927-932
          (expert_gate[:, :, i] * out_flat)[..., None, None]
          * one_hot(idx_i, e_)[..., None]
          * one_hot(position.astype(np.int32), capacity))
  zeros_i = np.zeros((g_, s_), np.int32)
  out = dict(
      index_1=index_1, index_2=zeros_i, pos_1=pos_1, pos_2=zeros_i,
      kept_1=kept_1, kept_2=np.zeros((g_, s_), bool),
      gate_1=gate_1, gate_2=np.zeros((g_, s_), F32),
      fill=cum_tokens.astype(np.int32), taken_in_pass=rnd, topk_index=expert_index,
      loss=cast_act(loss, act_dtype)[()])                        # :937
  if dense:
    combine = cast_act(combine, act_dtype)                       # :936
    out["combine"] = combine
    out["dispatch"] = (combine != 0).astype(F32)                 # :938-939
  return out


# ----------------------------------------------------------------------------
# _expert_selection_gating  (transformer/moe.py:1057-1173)
# ----------------------------------------------------------------------------
def expert_selection_gating(logits, capacity, importance,
                            num_microbatches=None, act_dtype="float32",
                            normalize_by_num_experts_routed=True, dense=False):
  """Everything in _expert_selection_gating after the router projection, for
  the policies that draw no random numbers: every expert picks the `capacity`
  tokens of each group it likes best.

  The softmax runs over the GROUP dim (per expert, over tokens); tokens with
  importance 0 get -1e9 added to their logits first (moe.py:1094-1097).  A
  token may be chosen by several experts or by none; its combine weights are
  the chosen probabilities divided by max(#experts that chose it, 1)
  (moe.py:1119-1123).  `importance` is required, as in the reference, whose
  loss sums it (moe.py:1138-1140).

  Returns dict(slot_token int32 [G,E,C] (token of each slot), slot_weight
  float32 [G,E,C] (combine weight before the activation-dtype cast), loss,
  and with dense=True combine / dispatch [G,S,E,C]).
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  importance = np.asarray(importance, dtype=F32)
  logits = logits + ((importance == F32(0.0)).astype(F32) * F32(-1e9))[..., None]
  # softmax over the group dim (ops.py:5493-5541 with reduced_dim = group)
  raw_gates = np.moveaxis(softmax(np.moveaxis(logits, 1, -1)), -1, 1)  # [G,S,E]
  probs, tokens = top_k_lowest_index_first(raw_gates, capacity, 1)    # [G,E,C]
  dispatch = one_hot(tokens, s_)                                 # [G,E,C,S]
  combine = dispatch * probs[..., None]                          # :1115
  slot_weight = probs
  if normalize_by_num_experts_routed:                            # :1119-1123
    num_routed = dispatch.sum(axis=(1, 2), dtype=F32)            # [G,S]
    recip = (F32(1.0) / np.maximum(num_routed, F32(1.0))).astype(F32)
    combine = combine * recip[:, None, None, :]
    slot_weight = probs * np.take_along_axis(
        recip[:, None, :].repeat(e_, 1), tokens, -1)
  # load balancing loss (:1125-1147)
  agg = seq_sum(raw_gates, axis=-1) * F32(1.0 / e_)              # [G,S]
  agg = agg * (importance == F32(1.0)).astype(F32)
  true_group_size = seq_sum(importance, axis=-1)                 # [G]
  prod = (agg * agg) * true_group_size[:, None]
  loss = seq_sum(prod.reshape(-1)) * F32(1.0 / prod.size)
  loss = loss * F32(float(s_))
  if num_microbatches and num_microbatches > 1:
    loss = loss * F32(1.0 / num_microbatches)
  out = dict(slot_token=tokens, slot_weight=slot_weight.astype(F32),
             loss=cast_act(loss, act_dtype)[()])
  if dense:
    out["combine"] = cast_act(combine.transpose(0, 3, 1, 2), act_dtype)
    out["dispatch"] = dispatch.transpose(0, 3, 1, 2).astype(F32)  # :1169-1170
  return out


# ----------------------------------------------------------------------------
# training-time scalar summaries of the f1 routers
# ----------------------------------------------------------------------------
def router_summaries(logits, gating, routing, importance=None, top_k=1,
                     num_microbatches=None, act_dtype="float32", capacity=None):
  """The values _switch_gating (moe.py:1213, :1242-1257, :1259-1269,
  :1285-1289), _switch_max_gating (:981, :1010-1025, :1041-1046), _ntlb_gating
  (:865-880) and _expert_selection_gating (:1149-1165) pass to
  mtf.scalar_summary while training, from the router's logits [G,S,E] and the
  gating function's result dict `routing`.

  Returns a dict: "entropy"; for the per-token routers "expert_gate" (mean
  largest probability, before the importance mask), "experts" [E] (share of
  every expert among the choices of importance-1 tokens), for the switch
  routers "fraction_routed" and "z_loss" (the value; the reference emits it
  only with moe_z_loss set); for expert selection "group_token" [S].  Sums over
  many terms accumulate in float64 and round once (the order of TensorFlow's
  reductions is not pinned).
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  eps = F32(1e-9)
  if gating == "expert_selection":
    importance = np.asarray(importance, dtype=F32)
    lg = logits + ((importance == F32(0.0)).astype(F32) * F32(-1e9))[..., None]
    raw = np.moveaxis(softmax(np.moveaxis(lg, 1, -1)), -1, 1)    # [G,S,E]
    terms = (-raw * np.log(raw + eps).astype(F32)).astype(F32)   # :1149
    entropy = terms.sum(axis=1, dtype=np.float64)                # [G,E]
    tokens = np.asarray(routing["slot_token"])                   # [G,E,C]
    cap = tokens.shape[-1]
    sent = np.zeros((s_,), np.float64)
    np.add.at(sent, tokens.reshape(-1), 1.0)                     # :1155-1158
    return dict(entropy=F32(entropy.mean()),
                group_token=(sent * float(e_ * cap)).astype(F32))
  raw = router_softmax(logits, gating, act_dtype)
  terms = (-raw * np.log(raw + eps).astype(F32)).astype(F32)
  entropy = F32(terms.sum(axis=-1, dtype=np.float64).mean())
  k_ = int(top_k) if gating == "ntlb" else 1
  gate, index = top_k_lowest_index_first(raw, k_, -1)            # [G,S,k]
  mask = one_hot(index, e_)                                      # [G,S,k,E]
  is_one = np.ones((g_, s_), F32)
  imp = np.ones((g_, s_), F32)
  if importance is not None:
    imp = np.asarray(importance, dtype=F32)
    is_one = (imp == F32(1.0)).astype(F32)
    mask = mask * is_one[..., None, None]
  counts = mask.sum(axis=(0, 1, 2), dtype=np.float64)            # [E]
  out = dict(entropy=entropy,
             expert_gate=F32(gate[..., 0].mean(dtype=np.float64)),
             experts=(counts / counts.sum()).astype(F32))
  if gating in ("switch", "switch_max"):
    kept = np.asarray(routing["kept_1"])
    out["fraction_routed"] = F32(kept.sum(dtype=np.float64) /
                                 imp.sum(dtype=np.float64))
    m = logits.max(axis=-1, keepdims=True)
    log_z = np.log(seq_sum(np.exp(logits + (-m)).astype(F32), axis=-1)
                   ).astype(F32) + m[..., 0]
    z = ((log_z * log_z) * is_one).sum(dtype=np.float64)
    out["z_loss"] = F32(z / (is_one.sum(dtype=np.float64) *
                             float(num_microbatches or 1)))
  return out


def slot_dispatch(x, r):
  """expert_in[e, g, c, :] = x[g, slot_token[g, e, c], :] (the dispatch einsum
  with a one-hot per slot, moe.py:443-447)."""
  g_ = x.shape[0]
  tok = r["slot_token"]                                          # [G,E,C]
  return x[np.arange(g_)[:, None, None], tok].transpose(1, 0, 2, 3)


def slot_combine(y, r, group_size, act_dtype):
  """out[g, s, :] = sum over the slots holding token s of w * y[e, g, c, :]
  with w the activation-dtype combine weight (moe.py:509-510); float32
  accumulate in (expert, slot) order, one rounding."""
  e_, g_, c_, n_ = y.shape
  w = cast_act(r["slot_weight"], act_dtype)
  out = np.zeros((g_, group_size, n_), F32)
  for g in range(g_):
    for e in range(e_):
      np.add.at(out[g], r["slot_token"][g, e], w[g, e][:, None] * y[e, g])
  return cast_act(out, act_dtype)


def routing_sequential(index_1, index_2, sel_1, sel_2, num_experts, capacity):
  """Integer brute force for moe.py:1472-1496, one token at a time.

  sel_k[g, s] says whether token s enters the k-th choice competition (mask_k
  before capacity).  Per group: first choices claim slots in token order; a
  first choice whose running count has reached `capacity` is dropped; second
  choices then claim slots starting from the kept first-choice count, and the
  running second-choice counter advances for every selected second choice,
  kept or not.

  Returns pos_1, kept_1, pos_2, kept_2, fill ([G,E] occupied slots).
  """
  g_, s_ = index_1.shape
  pos_1 = np.zeros((g_, s_), np.int32)
  pos_2 = np.zeros((g_, s_), np.int32)
  kept_1 = np.zeros((g_, s_), bool)
  kept_2 = np.zeros((g_, s_), bool)
  fill = np.zeros((g_, num_experts), np.int32)
  for g in range(g_):
    seen = [0] * num_experts
    for s in range(s_):
      if sel_1[g, s]:
        e = int(index_1[g, s])
        pos_1[g, s] = seen[e]
        kept_1[g, s] = seen[e] < capacity
        seen[e] += 1
    count_1 = [min(c, capacity) for c in seen]
    seen2 = [0] * num_experts
    kept2_count = [0] * num_experts
    for s in range(s_):
      if sel_2[g, s]:
        e = int(index_2[g, s])
        p = seen2[e] + count_1[e]
        pos_2[g, s] = p
        kept_2[g, s] = p < capacity
        kept2_count[e] += int(p < capacity)
        seen2[e] += 1
    for e in range(num_experts):
      fill[g, e] = count_1[e] + kept2_count[e]
  return pos_1, kept_1, pos_2, kept_2, fill


# ----------------------------------------------------------------------------
# index-form dispatch / combine (what the HIP kernels compute)
# ----------------------------------------------------------------------------
def combine_weights(r, act_dtype):
  """The two per-token combine weights as the dense tensor holds them: gate_k
  (already multiplied by mask_k_flat) cast to the activation dtype
  (moe.py:1499-1507)."""
  return cast_act(r["gate_1"], act_dtype), cast_act(r["gate_2"], act_dtype)


def dispatch_gather(x, r, num_experts, capacity, act_dtype):
  """expert_in[e, g, c, :] from the routing record; equals the dense einsum at
  moe.py:443-447 because each slot receives at most one token.  A kept choice
  whose activation-dtype gate is exactly zero is not dispatched
  (moe.py:1510-1511)."""
  g_, s_, m_ = x.shape
  w1, w2 = combine_weights(r, act_dtype)
  out = np.zeros((num_experts, g_, capacity, m_), F32)
  for k, w in (("1", w1), ("2", w2)):
    sel = r["kept_" + k] & (w != 0)
    gi, si = np.nonzero(sel)
    out[r["index_" + k][gi, si], gi, r["pos_" + k][gi, si]] = x[gi, si]
  return out


def combine_gather(y, r, act_dtype):
  """out[g, s, :] = w1 * y[idx1, g, pos1] + w2 * y[idx2, g, pos2]
  (moe.py:509-510 with at most two non-zero terms), float32 accumulate, one
  rounding to the activation dtype."""
  e_, g_, c_, n_ = y.shape
  w1, w2 = combine_weights(r, act_dtype)
  s_ = w1.shape[1]
  out = np.zeros((g_, s_, n_), F32)
  for k, w in (("1", w1), ("2", w2)):
    sel = r["kept_" + k] & (w != 0)
    gi, si = np.nonzero(sel)
    out[gi, si] += (w[gi, si][:, None]
                    * y[r["index_" + k][gi, si], gi, r["pos_" + k][gi, si]])
  return cast_act(out, act_dtype)


# ----------------------------------------------------------------------------
# activations (ops.py:1818-1921)
# ----------------------------------------------------------------------------
def _gelu(x):
  # ops.py:1862-1874: 0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 x^3)))
  x = x.astype(F32)
  cdf = F32(0.5) * (F32(1.0) + np.tanh(
      F32(np.sqrt(2 / np.pi)) * (x + F32(0.044715) * x * x * x)).astype(F32))
  return x * cdf


ACTIVATIONS = {
    "relu": lambda x: np.maximum(x, F32(0)),
    "linear": lambda x: x,
    None: lambda x: x,
    "gelu": _gelu,
    "sigmoid": lambda x: (F32(1) / (F32(1) + np.exp(-x))).astype(F32),
    "tanh": lambda x: np.tanh(x).astype(F32),
    "swish": lambda x: (x / (F32(1) + np.exp(-x))).astype(F32),
}


# ----------------------------------------------------------------------------
# the layers
# ----------------------------------------------------------------------------
class HParams(object):
  """Attribute bag (transformer/moe.py:1585-1596)."""

  def __init__(self, **kwargs):
    for k, v in kwargs.items():
      setattr(self, k, v)


def default_hparams(**overrides):
  hp = dict(
      moe_gating="top_2", moe_num_experts=16, moe_loss_coef=1e-2,
      moe_hidden_size=4096, moe_group_size=1024, moe_min_expert_capacity=4,
      moe_capacity_factor_train=1.25, moe_capacity_factor_eval=2.0,
      moe_capacity_factor_second_level=1.0,
      moe_use_second_place_loss=False,
      moe_second_policy_train="random", moe_second_policy_eval="random",
      moe_second_threshold_train=0.2, moe_second_threshold_eval=0.2,
      moe_dropout_rate=0.0, moe_use_experts_attention=False,
      moe_switch_policy_train="input_jitter",
      moe_switch_policy_eval="input_jitter", moe_switch_dropout=0.1,
      moe_switch_temperature=1.0, moe_switch_jitter=1e-2, moe_z_loss=None,
      moe_ntlb_top_k=4)
  hp.update(overrides)
  return HParams(**hp)


def router_logits(x, w):
  """raw_gates = dense(to_float(inputs), experts_dim, use_bias=False)
  (moe.py:1384-1390; layers.py:129-208, einsum in float32).  x [..., M] and
  w [M, E] already hold activation-dtype-rounded values (ops.py:4046-4047,
  layers.py:252)."""
  return np.matmul(x.astype(F32), w.astype(F32)).astype(F32)


def _policy(hp, train):
  if train:
    return hp.moe_second_policy_train, hp.moe_second_threshold_train
  return hp.moe_second_policy_eval, hp.moe_second_threshold_eval


def _scale_loss(loss, coef, act_dtype):
  """`loss * hparams.moe_loss_coef` on an activation-dtype scalar
  (moe.py:525; ScalarMultiplyOperation ops.py:2006-2023)."""
  return cast_act(cast_act(loss, act_dtype) * cast_act(F32(coef), act_dtype),
                  act_dtype)[()]


def hidden_dropout_noise(uniform, keep_prob, act_dtype):
  """mtf.dropout's multiplier (ops.py:5864-5872) for a tensor of the activation
  dtype: cast(uniform < keep_prob) / keep_prob, where `uniform` holds
  activation-dtype values in [0, 1) and keep_prob is a scalar of that dtype, so
  both it and the quotient are rounded to it."""
  keep = cast_act(F32(keep_prob), act_dtype)
  u = cast_act(np.asarray(uniform, F32), act_dtype)
  return cast_act((u < keep).astype(F32) / keep, act_dtype)


def expert_hidden(expert_in, wi, activation, act_dtype, hidden_noise=None):
  """The experts' hidden tensor (moe.py:469-479): the product over the factors
  of mtf.layers.dense_product (layers.py:279-295) of act_i(expert_in . wi_i),
  times the dropout noise.  wi / activation: one kernel [E, M, H] and one
  name, or lists of the same length.  Every op rounds to the activation dtype.
  """
  wis = list(wi) if isinstance(wi, (list, tuple)) else [wi]
  acts = (list(activation) if isinstance(activation, (list, tuple))
          else [activation])
  if len(wis) != len(acts):
    raise ValueError("%d kernels for %d activations" % (len(wis), len(acts)))
  h = None
  for w, a in zip(wis, acts):
    f = cast_act(np.matmul(expert_in, w), act_dtype)
    f = cast_act(ACTIVATIONS[a](f), act_dtype)
    h = f if h is None else cast_act(h * f, act_dtype)
  if hidden_noise is not None:
    h = cast_act(h * hidden_noise, act_dtype)
  return h


def expert_ffn(expert_in, wi, wo, activation, act_dtype, hidden_noise=None):
  """h = act(expert_in . wi), y = h . wo per expert (moe.py:469-486).
  expert_in [E, R, M], wi [E, M, H] (or a list, see expert_hidden),
  wo [E, H, N]; float32 accumulate, results rounded to the activation dtype.
  hidden_noise [E, R, H]: the dropout multiplier on h, if any."""
  h = expert_hidden(expert_in, wi, activation, act_dtype, hidden_noise)
  return cast_act(np.matmul(h, wo), act_dtype)


def perturb_gate_inputs(xg, hp, train, act_dtype, gate_noise):
  """The router's input under hparams.moe_switch_policy_*:

  _switch_gating / _expert_selection_gating (moe.py:1189-1199, :1071-1078):
  gate_inputs = to_float(inputs); "input_dropout" multiplies by
  (u < keep_prob) / keep_prob while training (mtf.dropout, ops.py:5864-5872),
  "input_jitter" by u in [1 - eps, 1 + eps) while training
  (mtf.layers.multiplicative_jitter, layers.py:1949-1952).
  _ntlb_gating (moe.py:821-822) knows only the jitter and applies it in the
  activation dtype.

  gate_noise stands in for the random tensor u ~ U[0, 1) of xg's shape (the
  reference draws it from TensorFlow's generator).  Returns (gate inputs,
  the multiplier or None).
  """
  policy = hp.moe_switch_policy_train if train else hp.moe_switch_policy_eval
  ntlb = hp.moe_gating == "ntlb"
  jitter = train and policy == "input_jitter"
  dropout = train and policy == "input_dropout" and not ntlb
  if not (jitter or dropout):
    return xg, None
  if gate_noise is None:
    raise NotImplementedError(
        "switch policy %r needs the random tensor (gate_noise)" % policy)
  u = np.asarray(gate_noise, F32).reshape(xg.shape)
  if jitter:
    eps = F32(hp.moe_switch_jitter)
    if ntlb:       # random_uniform(dtype = activation dtype), product rounded
      mult = cast_act((F32(1.0) - eps) + u * (F32(2.0) * eps), act_dtype)
      return cast_act(xg * mult, act_dtype), mult
    mult = (F32(1.0) - eps) + u * (F32(2.0) * eps)
    return (xg.astype(F32) * mult).astype(F32), mult
  keep = F32(1.0 - hp.moe_switch_dropout)
  mult = (u < keep).astype(F32) / keep
  return (xg.astype(F32) * mult).astype(F32), mult


def _cast_kernels(w, act_dtype):
  if isinstance(w, (list, tuple)):
    return [cast_act(v, act_dtype) for v in w]
  return cast_act(w, act_dtype)


def moe_layer_v1(x, w_gate, wi, wo, hp, train, act_dtype="float32",
                 nonpadding=None, activation="relu", num_microbatches=None,
                 logit_bias=None, second_uniform=None, dense=True,
                 mesh_dim_size=1, weights_are_cast=False, k_wo=None,
                 gate_noise=None, sample_uniform=None, hidden_uniform=None):
  """transformer_moe_layer_v1 forward (transformer/moe.py:191-525).

  x: [batch..., length, M] float32 array holding activation-dtype values.
  w_gate [M, E], wi [E, M, H], wo [E, H, N]: master (float32) weights; they are
  cast to the activation dtype as Variable.lower does (ops.py:4046-4047).
  logit_bias: optional [E] added to the router logits (benchmark-only hook for
  the skewed-routing config; the reference router has no bias).
  dense=True follows the reference dataflow literally (one-hot [G,S,E,C]
  tensors, einsums); dense=False uses the index form.
  k_wo [E, H, N]: with hparams.moe_use_experts_attention `wo` is the "q_wo"
  kernel and k_wo the "k_wo" kernel of a second output projection of the same
  hidden tensor (moe.py:514-522); the output is then the list [q, k].
  wi / activation may be lists of the same length (gated units, see
  expert_hidden).  hidden_uniform [E, G*C, H]: the uniform numbers of the
  dropout on the hidden tensor, needed when train and hp.moe_dropout_rate != 0
  (moe.py:477-479).

  Returns (output [batch..., length, N], loss scalar, aux dict).
  """
  if getattr(hp, "moe_use_experts_attention", False):
    if k_wo is None:
      raise ValueError("moe_use_experts_attention needs the k_wo kernel")
    import copy
    hp1 = copy.copy(hp)
    hp1.moe_use_experts_attention = False
    kw = dict(nonpadding=nonpadding, activation=activation,
              num_microbatches=num_microbatches, logit_bias=logit_bias,
              second_uniform=second_uniform, dense=dense,
              mesh_dim_size=mesh_dim_size, weights_are_cast=weights_are_cast,
              gate_noise=gate_noise, sample_uniform=sample_uniform,
              hidden_uniform=hidden_uniform)
    # the two outputs share everything up to the hidden tensor, so each equals
    # the plain layer with its own output kernel
    q, loss, aux = moe_layer_v1(x, w_gate, wi, wo, hp1, train, act_dtype, **kw)
    k, _, _ = moe_layer_v1(x, w_gate, wi, k_wo, hp1, train, act_dtype, **kw)
    return [q, k], loss, aux
  if hp.moe_gating not in ("top_2", "switch", "switch_max", "ntlb",
                          "expert_selection"):
    raise ValueError("unknown hparams.moe_gating=%s" % hp.moe_gating)
  x = cast_act(x, act_dtype)
  lead = x.shape[:-1]
  m_ = x.shape[-1]
  n_tok = int(np.prod(lead))
  e_ = hp.moe_num_experts
  g_, s_ = split_into_groups(n_tok, hp.moe_group_size, mesh_dim_size)
  cf = hp.moe_capacity_factor_train if train else hp.moe_capacity_factor_eval
  c_ = expert_capacity(s_, cf, e_, hp.moe_min_expert_capacity)
  xg = x.reshape(g_, s_, m_)                                     # :359-361
  importance = None
  if nonpadding is not None:                                     # :376-379
    importance = cast_act(np.broadcast_to(nonpadding, lead), act_dtype)
    importance = importance.reshape(g_, s_)
  wg = cast_act(w_gate, act_dtype)
  hidden_noise = None
  if train and getattr(hp, "moe_dropout_rate", 0.0) != 0.0:
    if hidden_uniform is None:
      raise NotImplementedError(
          "moe_dropout_rate while training needs the random tensor "
          "(hidden_uniform)")
    hidden_noise = hidden_dropout_noise(
        hidden_uniform, 1.0 - hp.moe_dropout_rate, act_dtype)
  gate_mult = None
  if hp.moe_gating in ("switch", "switch_max", "ntlb", "expert_selection"):
    x_gate, gate_mult = perturb_gate_inputs(xg, hp, train, act_dtype,
                                            gate_noise)
    logits = router_logits(x_gate, wg)
  else:
    logits = router_logits(xg, wg)
  if logit_bias is not None:
    logits = logits + np.asarray(logit_bias, F32)
  if hp.moe_gating == "expert_selection":                        # :425-438
    if importance is None:
      raise ValueError("expert_selection gating needs nonpadding "
                       "(moe.py:1138-1140)")
    r = expert_selection_gating(logits, c_, importance, num_microbatches,
                                act_dtype, dense=dense)
    wi_a = wi if weights_are_cast else _cast_kernels(wi, act_dtype)
    wo_a = wo if weights_are_cast else cast_act(wo, act_dtype)
    if dense:
      disp = r["dispatch"].reshape(g_, s_, e_ * c_)
      expert_in = cast_act(np.matmul(disp.transpose(0, 2, 1), xg), act_dtype)
      expert_in = expert_in.reshape(g_, e_, c_, m_).transpose(1, 0, 2, 3)
    else:
      expert_in = slot_dispatch(xg, r)
    y = expert_ffn(expert_in.reshape(e_, g_ * c_, m_), wi_a, wo_a, activation,
                   act_dtype, hidden_noise)
    n_ = y.shape[-1]
    y = y.reshape(e_, g_, c_, n_)
    if dense:
      comb = r["combine"].reshape(g_, s_, e_ * c_)
      yg = y.transpose(1, 0, 2, 3).reshape(g_, e_ * c_, n_)
      out = cast_act(np.matmul(comb, yg), act_dtype)
    else:
      out = slot_combine(y, r, s_, act_dtype)
    aux = dict(r, logits=logits, expert_in=expert_in, expert_out=y,
               num_groups=g_, group_size=s_, capacity=c_, gate_mult=gate_mult)
    return (out.reshape(lead + (n_,)),
            _scale_loss(r["loss"], hp.moe_loss_coef, act_dtype), aux)
  if hp.moe_gating in ("switch", "switch_max", "ntlb"):          # :393-424
    sw = hp.moe_switch_policy_train if train else hp.moe_switch_policy_eval
    if sw not in ("argmax", "input_dropout", "input_jitter", "sample"):
      raise ValueError("Unknown Switch gating policy %s" % sw)
    choice = None
    if sw == "sample" and hp.moe_gating != "ntlb" and (
        hp.moe_switch_temperature != 0.0):
      if sample_uniform is None:
        raise NotImplementedError(
            "switch policy 'sample' needs the random tensor (sample_uniform)")
      choice = sample_choice_logits(
          logits, hp.moe_switch_temperature,
          np.asarray(sample_uniform, F32).reshape(logits.shape))
    if hp.moe_gating == "switch":
      r = switch_gating(logits, c_, importance, train, hp.moe_z_loss,
                        num_microbatches, act_dtype, dense=dense,
                        choice_logits=choice)
    elif hp.moe_gating == "ntlb":
      r = ntlb_gating(logits, c_, hp.moe_ntlb_top_k, importance,
                      num_microbatches, act_dtype, dense=dense)
    else:
      r = switch_max_gating(logits, c_, importance, num_microbatches,
                            act_dtype, dense=dense, choice_logits=choice)
  else:
    policy, threshold = _policy(hp, train)
    r = top_2_gating(logits, c_, importance, policy, threshold,
                     hp.moe_use_second_place_loss, num_microbatches, act_dtype,
                     second_uniform, dense=dense)
  # weights_are_cast: the caller already holds activation-dtype values (lets
  # the CPU-baseline timing pass one expert's matrix broadcast to all experts)
  wi_a = wi if weights_are_cast else _cast_kernels(wi, act_dtype)
  wo_a = wo if weights_are_cast else cast_act(wo, act_dtype)
  if dense:
    disp = r["dispatch"].reshape(g_, s_, e_ * c_)
    expert_in = np.matmul(disp.transpose(0, 2, 1), xg)           # [G, EC, M]
    expert_in = cast_act(expert_in, act_dtype).reshape(g_, e_, c_, m_)
    expert_in = expert_in.transpose(1, 0, 2, 3)                  # [E,G,C,M]
  else:
    expert_in = dispatch_gather(xg, r, e_, c_, act_dtype)
  y = expert_ffn(expert_in.reshape(e_, g_ * c_, m_), wi_a, wo_a, activation,
                 act_dtype, hidden_noise)
  n_ = y.shape[-1]
  y = y.reshape(e_, g_, c_, n_)
  if dense:
    comb = r["combine"].reshape(g_, s_, e_ * c_)
    yg = y.transpose(1, 0, 2, 3).reshape(g_, e_ * c_, n_)
    out = cast_act(np.matmul(comb, yg), act_dtype)               # :509-510
  else:
    out = combine_gather(y, r, act_dtype)
  aux = dict(r, logits=logits, expert_in=expert_in, expert_out=y,
             num_groups=g_, group_size=s_, capacity=c_, gate_mult=gate_mult)
  return (out.reshape(lead + (n_,)),
          _scale_loss(r["loss"], hp.moe_loss_coef, act_dtype), aux)


# ----------------------------------------------------------------------------
# backward of transformer_moe_layer_v1
# ----------------------------------------------------------------------------
def gating_backward(logits, r, gating, d_gate_1, d_gate_2, d_loss,
                    importance=None, num_microbatches=None, z_loss=None,
                    use_second_place_loss=False, act_dtype="float32"):
  """d(logits) of _top_2_gating / _switch_gating / _switch_max_gating /
  _ntlb_gating.

  The reference obtains it from the gradients of the ops the gating is built
  from: top_1 routes the gradient of a gate to the arg-max entry
  (TopKOperation.gradient, ops.py:4916-4920); one_hot, cumsum-of-masks,
  comparisons and the bool cast that makes the dispatch tensor have no
  gradient; divide/add/multiply are the usual rules (ops.py:2044-2084);
  softmax = exp(x - logsumexp(x)) (ops.py:5493-5541).

  d_gate_k [G,S]: gradient w.r.t. the combine weight gate_k * mask_k_flat
  (float32, zero where not kept); d_loss: gradient w.r.t. the balancing loss
  before moe_loss_coef.  Returns float32 [G,S,E].

  act_dtype matters for "ntlb" only: with "bfloat16" the probabilities are the
  bfloat16 softmax's (router_softmax), and the derivative below is the float32
  formula evaluated at them (the reference's own chain through the bfloat16
  ops rounds after each of them; the difference is inside the bfloat16
  tolerance of the layer's gradients).
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  p = router_softmax(logits, gating, act_dtype)
  rows = np.arange(g_)[:, None], np.arange(s_)[None, :]
  i1 = r["index_1"]
  one = np.ones((g_, s_), F32)
  m1 = one if importance is None else (
      np.asarray(importance, F32) == F32(1.0)).astype(F32)
  mb = F32(1.0 / num_microbatches) if (num_microbatches and
                                       num_microbatches > 1) else F32(1.0)
  dp = np.zeros_like(p)
  d_loss = F32(d_loss)
  inv_s = F32(1.0 / s_)
  ee = F32(float(e_ * e_))
  if gating == "top_2":
    i2 = r["index_2"]
    g1 = p[rows + (i1,)] * m1
    same = (i2 == i1).astype(F32) * m1
    g2 = p[rows + (i2,)] * (one - same)
    dg1n = np.asarray(d_gate_1, F32) * r["kept_1"]
    dg2n = np.asarray(d_gate_2, F32) * r["kept_2"]
    rec = F32(1.0) / ((g1 + g2) + F32(1e-9))                     # moe.py:1413
    common = (dg1n * g1 + dg2n * g2) * rec * rec
    dg1 = dg1n * rec - common
    dg2 = dg2n * rec - common
    np.add.at(dp, rows + (i1,), dg1 * m1)
    np.add.at(dp, rows + (i2,), dg2 * (one - same))
    # loss = mean_{g,e}(mean_s(p * m1) * density_1) * E^2   (moe.py:1420-1424)
    density = seq_sum(one_hot(i1, e_) * m1[..., None], axis=-2) * inv_s
    coef = d_loss * mb * ee * F32(1.0 / (g_ * e_))
    dp += (coef * density * inv_s)[:, None, :] * m1[..., None]
    if use_second_place_loss:
      # loss_2 * 0.5 = 0.5 E^2 mean_{g,e}(mean_s(n) * density_2), n = q /
      # (sum_e q + 1e-9), q = p * (1 - mask_1) (moe.py:1405, :1426-1438);
      # density_2 counts mask_2 before the second-choice policy and has no
      # gradient
      keep = one[..., None] - one_hot(i1, e_) * m1[..., None]
      q = p * keep
      m2 = one if importance is None else (
          np.asarray(importance, F32) > F32(0.0)).astype(F32)
      density_2 = seq_sum(one_hot(i2, e_) * m2[..., None], axis=-2) * inv_s
      a = (coef * F32(0.5) * density_2 * inv_s)[:, None, :]     # d/dn [G,1,E]
      rq = F32(1.0) / (q.sum(-1, keepdims=True) + F32(1e-9))
      dq = a * rq - (a * q).sum(-1, keepdims=True) * rq * rq
      dp += dq * keep
    return (p * (dp - (p * dp).sum(-1, keepdims=True))).astype(F32)
  if gating not in ("switch", "switch_max", "ntlb"):
    raise ValueError("unknown gating %r" % (gating,))
  # index_1 is the expert that took the token: the arg-max (switch) or the
  # candidate of the pass that placed it (ntlb: mtf.top_k routes the gradient
  # of each value to its entry, ops.py:4916-4920, :5009-5015)
  np.add.at(dp, rows + (i1,), np.asarray(d_gate_1, F32) * r["kept_1"] * m1)
  # loss = mean(mean_s(p)[g,e] * m1[g,s] * density_1[g,e]) * E^2 with density_1
  # counting every token (moe.py:1224-1234); ntlb has one density per pass and
  # the mean runs over the passes too (moe.py:845-856)
  if gating == "ntlb":
    k_ = r["topk_index"].shape[-1]
    density = seq_sum(one_hot(r["topk_index"], e_).sum(axis=2, dtype=F32),
                      axis=-2) * inv_s
    terms = g_ * e_ * k_
  else:
    density = seq_sum(one_hot(i1, e_), axis=-2) * inv_s
    terms = g_ * e_
  if importance is None:
    coef = d_loss * mb * ee * F32(1.0 / terms)
    dproxy = coef * density
  else:
    coef = d_loss * mb * ee * F32(1.0 / (terms * s_))
    dproxy = coef * density * m1.sum(-1, dtype=F32)[:, None]
  dp += (dproxy * inv_s)[:, None, :]
  dlogits = p * (dp - (p * dp).sum(-1, keepdims=True))
  if z_loss is not None:                                        # moe.py:1253-1266
    m = logits.max(-1, keepdims=True)
    lse = (np.log(np.exp(logits - m).sum(-1)) + m[..., 0]).astype(F32)
    denom = m1.sum(dtype=F32) * F32(num_microbatches)
    dlogits = dlogits + ((d_loss * F32(z_loss) * F32(2.0)) * lse * m1
                         / denom)[..., None] * p
  return dlogits.astype(F32)


def expert_selection_gating_backward(logits, r, importance, d_slot_weight,
                                     d_loss, num_microbatches=None,
                                     normalize_by_num_experts_routed=True):
  """d(logits) of _expert_selection_gating (moe.py:1094-1147).

  The probabilities are a softmax over the GROUP's tokens, one column per
  expert.  A slot's combine weight is the probability it was chosen with over
  max(#experts that chose the token, 1); top_k routes the gradient of a chosen
  value to its entry (ops.py:4916-4920, :5009-5015), the count comes from
  one-hot tensors and has no gradient.  The loss mean(agg^2 * sum(importance))
  * S with agg = mean_e p * (importance == 1) differentiates through agg.

  d_slot_weight [G,E,C]: gradient w.r.t. the float32 combine weight of each
  slot; d_loss: gradient w.r.t. the loss before moe_loss_coef.  Returns float32
  [G,S,E].
  """
  logits = np.asarray(logits, dtype=F32)
  g_, s_, e_ = logits.shape
  importance = np.asarray(importance, dtype=F32)
  masked = logits + ((importance == F32(0.0)).astype(F32) * F32(-1e9))[..., None]
  p = np.moveaxis(softmax(np.moveaxis(masked, 1, -1)), -1, 1)    # [G,S,E]
  tok = r["slot_token"]                                          # [G,E,C]
  gi = np.arange(g_)[:, None, None]
  ei = np.arange(e_)[None, :, None]
  recip = np.ones((g_, s_), F32)
  if normalize_by_num_experts_routed:
    num_routed = np.zeros((g_, s_), F32)
    np.add.at(num_routed, (np.broadcast_to(gi, tok.shape), tok), F32(1.0))
    recip = (F32(1.0) / np.maximum(num_routed, F32(1.0))).astype(F32)
  dp = np.zeros_like(p)
  dp[gi, tok, ei] = np.asarray(d_slot_weight, F32) * recip[gi, tok]
  is_one = (importance == F32(1.0)).astype(F32)
  agg = p.sum(-1, dtype=F32) * F32(1.0 / e_) * is_one
  tgs = importance.sum(-1, dtype=F32)                            # [G]
  mb = F32(1.0 / num_microbatches) if (num_microbatches and
                                       num_microbatches > 1) else F32(1.0)
  dagg = F32(d_loss) * mb * F32(2.0 / g_) * agg * tgs[:, None]
  dp += (dagg * is_one * F32(1.0 / e_))[..., None]
  return (p * (dp - (p * dp).sum(1, keepdims=True))).astype(F32)


def slot_combine_backward(dout, y, r, act_dtype):
  """Backward of the combine einsum for a per-slot record: dy [E,G,C,N] =
  w * dout[token of the slot] (activation dtype), d_slot_weight [G,E,C] =
  <dout[token], y[slot]> (float32)."""
  e_, g_, c_, _ = y.shape
  w = cast_act(r["slot_weight"], act_dtype)                      # [G,E,C]
  rows = dout[np.arange(g_)[:, None, None], r["slot_token"]]     # [G,E,C,N]
  dy = cast_act(w[..., None] * rows, act_dtype).transpose(1, 0, 2, 3)
  dw = (rows * y.transpose(1, 0, 2, 3)).sum(-1, dtype=F32)
  return dy, dw


def slot_dispatch_backward(dxe, r, group_size):
  """Backward of the dispatch einsum for a per-slot record: a token gathers
  the rows of all slots that hold it.  dxe [E,G,C,M] -> float32 [G,S,M]."""
  e_, g_, c_, m_ = dxe.shape
  dx = np.zeros((g_, group_size, m_), F32)
  for g in range(g_):
    for e in range(e_):
      np.add.at(dx[g], r["slot_token"][g, e], dxe[e, g].astype(F32))
  return dx


def combine_backward(dout, y, r, act_dtype):
  """Backward of the combine einsum (moe.py:509-510) in gather form.
  dout [G,S,N], y [E,G,C,N] -> dy [E,G,C,N] (activation dtype; zero rows for
  empty slots), dgate [G,S,2] float32 (zero where not kept)."""
  g_, s_, _ = dout.shape
  dy = np.zeros_like(y)
  dgate = np.zeros((g_, s_, 2), F32)
  for ki, (k, w) in enumerate(zip("12", combine_weights(r, act_dtype))):
    gi, si = np.nonzero(r["kept_" + k])
    ei, ci = r["index_" + k][gi, si], r["pos_" + k][gi, si]
    dgate[gi, si, ki] = (dout[gi, si] * y[ei, gi, ci]).sum(-1, dtype=F32)
    dy[ei, gi, ci] = cast_act(w[gi, si][:, None] * dout[gi, si], act_dtype)
  return dy, dgate


def dispatch_backward(dxe, r, act_dtype):
  """Backward of the dispatch einsum (moe.py:443-447): a token gathers the
  rows of the slots it was dispatched to.  dxe [E,G,C,M] -> float32 [G,S,M]
  (not yet rounded: the router's share is added before the cast)."""
  _, g_, _, m_ = dxe.shape
  s_ = r["kept_1"].shape[1]
  dx = np.zeros((g_, s_, m_), F32)
  for k, w in zip("12", combine_weights(r, act_dtype)):
    gi, si = np.nonzero(r["kept_" + k] & (w != 0))
    dx[gi, si] += dxe[r["index_" + k][gi, si], gi, r["pos_" + k][gi, si]]
  return dx


def _gelu_grad(x):
  k = F32(np.sqrt(2 / np.pi))
  t = np.tanh(k * (x + F32(0.044715) * x * x * x)).astype(F32)
  du = k * (F32(1.0) + F32(3 * 0.044715) * x * x)
  return F32(0.5) * (F32(1.0) + t) + F32(0.5) * x * (F32(1.0) - t * t) * du


def _sigmoid(x):
  return (F32(1) / (F32(1) + np.exp(-x))).astype(F32)


# d act(x) / dx from the pre-activation, float32
ACTIVATION_GRADS = {
    "relu": lambda x: (x > 0).astype(F32),
    "linear": lambda x: np.ones_like(x, dtype=F32),
    None: lambda x: np.ones_like(x, dtype=F32),
    "gelu": _gelu_grad,
    "sigmoid": lambda x: _sigmoid(x) * (F32(1) - _sigmoid(x)),
    "tanh": lambda x: F32(1) - np.tanh(x).astype(F32) ** 2,
    "swish": lambda x: _sigmoid(x) + x * _sigmoid(x) * (F32(1) - _sigmoid(x)),
}


def expert_ffn_backward(xe, wi_a, wo_a, dy, activation, act_dtype,
                        hidden_noise=None):
  """Backward of the expert einsums (moe.py:469-486): float32 accumulate,
  activation-dtype results.  xe [E,R,M], dy [E,R,N]; returns
  (dxe [E,R,M], dwi [E,M,H], dwo [E,H,N]).  hidden_noise [E,R,H]: the dropout
  multiplier on the hidden tensor (moe.py:477-479), a constant of the graph.

  wi_a / activation may be lists (a product of dense layers, layers.py:279-295;
  dwi is then a list): with f_i = act_i(pre_i), pre_i = xe . wi_i,
  h = noise * prod_i f_i, the gradient reaching pre_i is
  dh * noise * prod_{j != i} f_j * act_i'(pre_i); the derivative of an
  activation is taken in float32 from the (rounded) pre-activation and the
  product is rounded once (the reference differentiates the primitives an
  activation is built from, each rounding its result: a few more roundings in
  bfloat16, nothing else)."""
  is_list = isinstance(wi_a, (list, tuple))
  wis = list(wi_a) if is_list else [wi_a]
  acts = list(activation) if isinstance(activation, (list, tuple)) else [activation]
  if len(wis) != len(acts):
    raise ValueError("%d kernels for %d activations" % (len(wis), len(acts)))
  pres = [cast_act(np.matmul(xe, w), act_dtype) for w in wis]
  fs = [cast_act(ACTIVATIONS[a](p), act_dtype) for a, p in zip(acts, pres)]
  h = fs[0]
  for f in fs[1:]:
    h = cast_act(h * f, act_dtype)
  if hidden_noise is not None:
    h = cast_act(h * hidden_noise, act_dtype)
  dh = cast_act(np.matmul(dy, wo_a.transpose(0, 2, 1)), act_dtype)
  if hidden_noise is not None:
    dh = cast_act(dh * hidden_noise, act_dtype)
  dwo = cast_act(np.matmul(h.transpose(0, 2, 1), dy), act_dtype)
  dxe = np.zeros_like(xe, dtype=F32)
  dwis = []
  for i, (w, a, p) in enumerate(zip(wis, acts, pres)):
    g = dh
    for j, f in enumerate(fs):
      if j != i:
        g = cast_act(g * f, act_dtype)
    dpre = cast_act(g * ACTIVATION_GRADS[a](p), act_dtype)
    part = cast_act(np.matmul(dpre, w.transpose(0, 2, 1)), act_dtype)
    dxe = part if i == 0 else cast_act(dxe + part, act_dtype)
    dwis.append(cast_act(np.matmul(xe.transpose(0, 2, 1), dpre), act_dtype))
  return dxe, (dwis if is_list else dwis[0]), dwo


def moe_layer_v1_backward(x, w_gate, wi, wo, hp, train, act_dtype, d_out,
                          d_loss=0.0, nonpadding=None, activation="relu",
                          num_microbatches=None, logit_bias=None,
                          gate_noise=None, sample_uniform=None,
                          hidden_uniform=None, k_wo=None):
  """Gradients of (outputs, loss) of moe_layer_v1 w.r.t. x and the three
  kernels, given d_out [batch..., length, N] and the scalar d_loss.

  Follows what mtf.gradients (ops.py:5254-5291) assembles from the layer's ops:
  the combine / dispatch einsums and the two expert einsums back-propagate as
  einsums with the same one-hot tensors (EinsumOperation.gradient,
  ops.py:2846-2854), i.e. as the gather / scatter of the routing record;
  gradients are tensors of the activation dtype (cast gradients cast back,
  ops.py:1945-1962), float32 inside the gating.  The dispatch tensor is a
  bool cast of the combine tensor and carries no gradient (moe.py:1510-1511).

  With hparams.moe_use_experts_attention (k_wo given, d_out = [d_q, d_k]) the
  two outputs are two plain layers that share everything but the output kernel
  (moe_layer_v1), so every shared gradient is the sum of the two layers'
  (mtf.gradients adds the gradients of a tensor's consumers, ops.py:5276-5283)
  and "dk_wo" is the second layer's dwo.

  Returns dict(dx, dw_gate, dwi, dwo) holding activation-dtype values.
  """
  if getattr(hp, "moe_use_experts_attention", False):
    import copy
    hp1 = copy.copy(hp)
    hp1.moe_use_experts_attention = False
    kw = dict(nonpadding=nonpadding, activation=activation,
              num_microbatches=num_microbatches, logit_bias=logit_bias,
              gate_noise=gate_noise, sample_uniform=sample_uniform,
              hidden_uniform=hidden_uniform)
    q = moe_layer_v1_backward(x, w_gate, wi, wo, hp1, train, act_dtype,
                              d_out[0], d_loss, **kw)
    k = moe_layer_v1_backward(x, w_gate, wi, k_wo, hp1, train, act_dtype,
                              d_out[1], 0.0, **kw)
    out = {n: cast_act(q[n] + k[n], act_dtype) for n in ("dx", "dw_gate")}
    out["dwi"] = ([cast_act(a + b, act_dtype) for a, b in zip(q["dwi"], k["dwi"])]
                  if isinstance(q["dwi"], list)
                  else cast_act(q["dwi"] + k["dwi"], act_dtype))
    out.update(dwo=q["dwo"], dk_wo=k["dwo"], aux=q["aux"])
    return out
  _, _, aux = moe_layer_v1(x, w_gate, wi, wo, hp, train, act_dtype,
                           nonpadding=nonpadding, activation=activation,
                           num_microbatches=num_microbatches,
                           logit_bias=logit_bias, dense=False,
                           gate_noise=gate_noise,
                           sample_uniform=sample_uniform,
                           hidden_uniform=hidden_uniform)
  hidden_noise = None
  if train and getattr(hp, "moe_dropout_rate", 0.0) != 0.0:
    hidden_noise = hidden_dropout_noise(
        hidden_uniform, 1.0 - hp.moe_dropout_rate, act_dtype)
  x = cast_act(x, act_dtype)
  lead, m_ = x.shape[:-1], x.shape[-1]
  g_, s_, c_ = aux["num_groups"], aux["group_size"], aux["capacity"]
  e_ = hp.moe_num_experts
  xg = x.reshape(g_, s_, m_)
  wg_a, wo_a = cast_act(w_gate, act_dtype), cast_act(wo, act_dtype)
  wi_a = _cast_kernels(wi, act_dtype)
  n_ = wo_a.shape[-1]
  dout = cast_act(np.asarray(d_out, F32), act_dtype).reshape(g_, s_, n_)
  y = aux["expert_out"]                                          # [E,G,C,N]
  expert_in = aux["expert_in"]                                   # [E,G,C,M]

  by_slot = hp.moe_gating == "expert_selection"
  if by_slot:
    dy, dgate = slot_combine_backward(dout, y, aux, act_dtype)
  else:
    dy, dgate = combine_backward(dout, y, aux, act_dtype)
  r_ = g_ * c_
  dxe, dwi, dwo = expert_ffn_backward(
      expert_in.reshape(e_, r_, m_), wi_a, wo_a, dy.reshape(e_, r_, n_),
      activation, act_dtype, hidden_noise)
  if by_slot:
    dx = slot_dispatch_backward(dxe.reshape(e_, g_, c_, m_), aux, s_)
  else:
    dx = dispatch_backward(dxe.reshape(e_, g_, c_, m_), aux, act_dtype)

  # gating and router backward
  importance = None
  if nonpadding is not None:
    importance = cast_act(np.broadcast_to(nonpadding, lead), act_dtype)
    importance = importance.reshape(g_, s_)
  z = hp.moe_z_loss if (train and hp.moe_gating == "switch") else None
  # the returned loss is aux * moe_loss_coef in the activation dtype
  d_aux = F32(cast_act(F32(d_loss), act_dtype)
              * cast_act(F32(hp.moe_loss_coef), act_dtype))
  if by_slot:
    dlogits = expert_selection_gating_backward(
        aux["logits"], aux, importance, dgate, d_aux, num_microbatches)
  else:
    dlogits = gating_backward(aux["logits"], aux, hp.moe_gating, dgate[..., 0],
                              dgate[..., 1], d_aux, importance,
                              num_microbatches, z, hp.moe_use_second_place_loss,
                              act_dtype)
  # the router saw the perturbed inputs x * mult (perturb_gate_inputs); the
  # multiplier is a constant of the graph
  mult = aux.get("gate_mult")
  x_gate = xg.astype(F32) if mult is None else (
      cast_act(xg * mult, act_dtype) if hp.moe_gating == "ntlb"
      else xg.astype(F32) * mult)
  dwg = np.matmul(x_gate.reshape(-1, m_).T.astype(F32),
                  dlogits.reshape(-1, e_)).astype(F32)
  dx_router = np.matmul(dlogits, wg_a.T.astype(F32))
  if mult is not None:
    dx_router = dx_router * mult
  dx = dx + dx_router
  return dict(dx=cast_act(dx, act_dtype).reshape(lead + (m_,)),
              dw_gate=cast_act(dwg, act_dtype), dwi=dwi, dwo=dwo,
              dlogits=dlogits, dgate=dgate, aux=aux)


def moe_layer_v2(x, w_outer, w_inner, wi, wo, hp, train, act_dtype="float32",
                 nonpadding=None, num_microbatches=None, second_uniform=None,
                 dense=True, mesh_dim_size=1):
  """transformer_moe_layer_v2 forward (transformer/moe.py:528-801).

  x: [a0?, b1, l, M]; w_outer [M, X]; w_inner [X, M, Y];
  wi [Y, X, M, H]; wo [Y, X, H, N] (moe.py:702-712, :743-753, :765-774).
  second_uniform: optional pair (outer [g1,s], inner [x,h0,t]).
  Returns (output, loss, aux).
  """
  if hp.moe_gating != "top_2":
    raise ValueError("unknown hparams.moe_gating=%s" % hp.moe_gating)
  x = cast_act(x, act_dtype)
  orig_shape = x.shape
  if x.ndim == 3:                                                # :641-644
    x = x[None]
  a0, b1, l_, m_ = x.shape
  x_e, y_e = hp.moe_num_experts
  g1, s_ = split_into_groups(b1 * l_, hp.moe_group_size, mesh_dim_size)
  cf = hp.moe_capacity_factor_train if train else hp.moe_capacity_factor_eval
  c_ = expert_capacity(s_, cf, x_e, hp.moe_min_expert_capacity)
  h0, t_ = split_into_groups(a0 * g1 * c_, hp.moe_group_size, mesh_dim_size)
  d_ = expert_capacity(t_, hp.moe_capacity_factor_second_level, y_e,
                       hp.moe_min_expert_capacity)
  policy, threshold = _policy(hp, train)
  u_outer, u_inner = second_uniform if second_uniform is not None else (None,
                                                                        None)
  xg = x.reshape(a0 * g1, s_, m_)                                # :695
  importance = None
  if nonpadding is not None:                                     # :638-640,:697
    importance = cast_act(np.broadcast_to(nonpadding, (a0, b1, l_)), act_dtype)
    importance = importance.reshape(a0 * g1, s_)

  # ---- outer level (:702-727)
  logits_x = router_logits(xg, cast_act(w_outer, act_dtype))
  rx = top_2_gating(logits_x, c_, importance, policy, threshold,
                    hp.moe_use_second_place_loss, num_microbatches, act_dtype,
                    u_outer, dense=dense)
  ag = a0 * g1
  if dense:
    disp = rx["dispatch"].reshape(ag, s_, x_e * c_)
    ein = cast_act(np.matmul(disp.transpose(0, 2, 1), xg), act_dtype)
    ein = ein.reshape(ag, x_e, c_, m_).transpose(1, 0, 2, 3)     # [x,ag,c,m]
    imp_w = seq_sum(rx["combine"], axis=1)                       # [ag,x,c]
    imp_w = cast_act(imp_w, act_dtype).transpose(1, 0, 2)        # [x,ag,c]
  else:
    ein = dispatch_gather(xg, rx, x_e, c_, act_dtype)
    w1, w2 = combine_weights(rx, act_dtype)
    imp_w = np.zeros((x_e, ag, c_), F32)
    for k, w in (("1", w1), ("2", w2)):
      gi, si = np.nonzero(rx["kept_" + k])
      imp_w[rx["index_" + k][gi, si], gi, rx["pos_" + k][gi, si]] = w[gi, si]
  imp2 = F32(0.5) * ((imp_w > F32(0.5)).astype(F32)
                     + (imp_w > F32(0.0)).astype(F32))           # :725-727
  imp2 = cast_act(imp2, act_dtype)

  # ---- inner level (:737-759); a0 is the group-ish dim being re-split
  inputs_y = ein.reshape(x_e, h0, t_, m_)
  imp2 = imp2.reshape(x_e, h0, t_)
  w_in = cast_act(w_inner, act_dtype)                            # [X, M, Y]
  logits_y = np.matmul(inputs_y.reshape(x_e, h0 * t_, m_), w_in).astype(F32)
  logits_y = logits_y.reshape(x_e * h0, t_, y_e)
  ry = top_2_gating(logits_y, d_, imp2.reshape(x_e * h0, t_), policy,
                    threshold, hp.moe_use_second_place_loss, num_microbatches,
                    act_dtype, u_inner, dense=dense)
  xin = inputs_y.reshape(x_e * h0, t_, m_)
  if dense:
    disp = ry["dispatch"].reshape(x_e * h0, t_, y_e * d_)
    ein_y = cast_act(np.matmul(disp.transpose(0, 2, 1), xin), act_dtype)
    ein_y = ein_y.reshape(x_e, h0, y_e, d_, m_).transpose(2, 0, 1, 3, 4)
  else:
    ein_y = dispatch_gather(xin, ry, y_e, d_, act_dtype)          # [y,xh,d,m]
    ein_y = ein_y.reshape(y_e, x_e, h0, d_, m_)

  # ---- experts (:765-774), weights [Y, X, ...]
  wi_a = cast_act(wi, act_dtype)
  wo_a = cast_act(wo, act_dtype)
  h_dim = wi_a.shape[-1]
  n_ = wo_a.shape[-1]
  yy = expert_ffn(ein_y.reshape(y_e * x_e, h0 * d_, m_),
                  wi_a.reshape(y_e * x_e, m_, h_dim),
                  wo_a.reshape(y_e * x_e, h_dim, n_), "relu", act_dtype)
  yy = yy.reshape(y_e, x_e * h0, d_, n_)

  # ---- inner combine (:784), regroup (:788-791), outer combine (:794)
  if dense:
    comb = ry["combine"].reshape(x_e * h0, t_, y_e * d_)
    yg = yy.transpose(1, 0, 2, 3).reshape(x_e * h0, y_e * d_, n_)
    out_y = cast_act(np.matmul(comb, yg), act_dtype)
  else:
    out_y = combine_gather(yy, ry, act_dtype)
  eo_x = out_y.reshape(x_e, ag, c_, n_)
  if dense:
    comb = rx["combine"].reshape(ag, s_, x_e * c_)
    yg = eo_x.transpose(1, 0, 2, 3).reshape(ag, x_e * c_, n_)
    out = cast_act(np.matmul(comb, yg), act_dtype)
  else:
    out = combine_gather(eo_x, rx, act_dtype)
  out = out.reshape(orig_shape[:-1] + (n_,))
  loss = cast_act(rx["loss"] + ry["loss"], act_dtype)            # :801
  aux = dict(outer=rx, inner=ry, capacity_x=c_, capacity_y=d_,
             groups_x=(g1, s_), groups_y=(h0, t_), importance_inner=imp2,
             importance_outer=importance, logits_outer=logits_x,
             logits_inner=logits_y, expert_in_x=ein, expert_in_y=ein_y,
             expert_out_y=yy, expert_out_x=eo_x)
  return out, _scale_loss(loss, hp.moe_loss_coef, act_dtype), aux


def moe_layer_v2_backward(x, w_outer, w_inner, wi, wo, hp, train, act_dtype,
                          d_out, d_loss=0.0, nonpadding=None,
                          num_microbatches=None):
  """Gradients of (outputs, loss) of moe_layer_v2 w.r.t. x and the four
  kernels: the v1 pieces applied twice, inner level first.  The importance of
  the inner level is a comparison of the slot weights (moe.py:725-727) and
  carries no gradient.  Returns dict(dx, dw_outer, dw_inner, dwi, dwo)."""
  _, _, aux = moe_layer_v2(x, w_outer, w_inner, wi, wo, hp, train, act_dtype,
                           nonpadding=nonpadding,
                           num_microbatches=num_microbatches, dense=False)
  x = cast_act(x, act_dtype)
  orig_shape = x.shape
  m_ = x.shape[-1]
  rx, ry = aux["outer"], aux["inner"]
  x_e, y_e = hp.moe_num_experts
  c_, d_ = aux["capacity_x"], aux["capacity_y"]
  h0, t_ = aux["groups_y"]
  ag, s_ = rx["kept_1"].shape
  xg = x.reshape(ag, s_, m_)
  wo_a, wi_a = cast_act(wo, act_dtype), cast_act(wi, act_dtype)
  w_out_a, w_in_a = cast_act(w_outer, act_dtype), cast_act(w_inner, act_dtype)
  h_dim, n_ = wi_a.shape[-1], wo_a.shape[-1]
  dout = cast_act(np.asarray(d_out, F32), act_dtype).reshape(ag, s_, n_)
  d_aux = F32(cast_act(F32(d_loss), act_dtype)
              * cast_act(F32(hp.moe_loss_coef), act_dtype))

  # outer combine, then inner combine
  d_eo_x, dgate_x = combine_backward(dout, aux["expert_out_x"], rx, act_dtype)
  d_out_y = d_eo_x.reshape(x_e * h0, t_, n_)
  dyy, dgate_y = combine_backward(d_out_y, aux["expert_out_y"], ry, act_dtype)
  # experts
  ein_y = aux["expert_in_y"].reshape(y_e * x_e, h0 * d_, m_)
  dein_y, dwi, dwo = expert_ffn_backward(
      ein_y, wi_a.reshape(y_e * x_e, m_, h_dim),
      wo_a.reshape(y_e * x_e, h_dim, n_), dyy.reshape(y_e * x_e, h0 * d_, n_),
      "relu", act_dtype)
  # inner gating, router and dispatch
  imp_in = aux["importance_inner"].reshape(x_e * h0, t_)
  dlogits_y = gating_backward(aux["logits_inner"], ry, "top_2",
                              dgate_y[..., 0], dgate_y[..., 1], d_aux, imp_in,
                              num_microbatches,
                              use_second_place_loss=hp.moe_use_second_place_loss)
  inputs_y = aux["expert_in_x"].reshape(x_e, h0 * t_, m_)
  dl_y = dlogits_y.reshape(x_e, h0 * t_, y_e)
  dw_inner = np.matmul(inputs_y.transpose(0, 2, 1).astype(F32), dl_y)
  dxin = dispatch_backward(dein_y.reshape(y_e, x_e * h0, d_, m_), ry, act_dtype)
  dxin = dxin.reshape(x_e, h0 * t_, m_) + np.matmul(
      dl_y, w_in_a.transpose(0, 2, 1).astype(F32))
  d_ein = cast_act(dxin, act_dtype).reshape(x_e, ag, c_, m_)
  # outer gating, router and dispatch
  dlogits_x = gating_backward(aux["logits_outer"], rx, "top_2",
                              dgate_x[..., 0], dgate_x[..., 1], d_aux,
                              aux["importance_outer"], num_microbatches,
                              use_second_place_loss=hp.moe_use_second_place_loss)
  dw_outer = np.matmul(xg.reshape(-1, m_).T.astype(F32),
                       dlogits_x.reshape(-1, x_e))
  dx = dispatch_backward(d_ein, rx, act_dtype) + np.matmul(
      dlogits_x, w_out_a.T.astype(F32))
  return dict(dx=cast_act(dx, act_dtype).reshape(orig_shape),
              dw_outer=cast_act(dw_outer, act_dtype),
              dw_inner=cast_act(dw_inner, act_dtype),
              dwi=dwi.reshape(wi_a.shape), dwo=dwo.reshape(wo_a.shape), aux=aux)
