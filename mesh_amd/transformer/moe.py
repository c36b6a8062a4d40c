"""Top-2 gated Mixture-of-Experts layers on HipMeshImpl.

Same entry points, argument order, defaults, dimension names, variable names
and error types as mesh_tensorflow/transformer/moe.py (MoE1D :37-128, MoE2D
:131-188, transformer_moe_layer_v1 :191-525, transformer_moe_layer_v2
:528-801, _split_into_groups :1549-1582, HParams :1585-1596).  Where the
reference expands the layer into ~100 graph primitives and dense one-hot
[G,S,E,C] tensors, each layer here is ONE Operation whose slice function calls
the HIP kernels: router -> top-2 gating -> dispatch -> expert FFN -> combine.

Built: moe_gating "top_2" (every second-place policy, the second-place loss),
"switch", "switch_max", "ntlb" and "expert_selection" with their switch
policies ("argmax", "sample", "input_jitter", "input_dropout"); nonpadding / importance; moe_use_experts_attention; float32 and
bfloat16; mtf.gradients over the v1 layer (top_2 / switch / switch_max / ntlb,
ReLU or linear experts) and the v2 layer.  Not built (they raise NotImplementedError):
expert dropout while training, gated (list) activations, gradients of the
expert_selection router, and a mesh with more than one device.
"""

import torch

from mesh_amd import layers as mtf_layers
from mesh_amd import moe_hip
from mesh_amd import ops as mtf
from mesh_amd.transformer import transformer

_OTHER_GATINGS = ()


class HParams(object):
  """Attribute bag standing in for tf.contrib.training.HParams."""

  def __init__(self, **kwargs):
    for k, v in kwargs.items():
      setattr(self, k, v)

  def add_hparam(self, k, v):
    setattr(self, k, v)


def set_default_moe_hparams(hparams):
  """Adds the reference's default MoE hyperparameters (moe.py:1516-1546)."""
  hparams.moe_num_experts = 16
  hparams.moe_loss_coef = 1e-2
  hparams.add_hparam("moe_gating", "top_2")
  hparams.add_hparam("moe_capacity_factor_train", 1.25)
  hparams.add_hparam("moe_capacity_factor_eval", 2.0)
  hparams.add_hparam("moe_capacity_factor_second_level", 1.0)
  hparams.add_hparam("moe_hidden_size", 4096)
  hparams.add_hparam("moe_group_size", 1024)
  hparams.add_hparam("moe_use_second_place_loss", 0)
  hparams.add_hparam("moe_second_policy_train", "random")
  hparams.add_hparam("moe_second_policy_eval", "random")
  hparams.add_hparam("moe_second_threshold_train", 0.2)
  hparams.add_hparam("moe_second_threshold_eval", 0.2)


def _split_into_groups(n, max_group_size, mesh_dim_size):
  """n = num_groups * group_size with group_size the largest value that is
  <= max_group_size and leaves num_groups a multiple of mesh_dim_size."""
  if n % mesh_dim_size != 0:
    raise ValueError(
        "n=%d is not a multiple of mesh_dim_size=%d" % (n, mesh_dim_size))
  num_groups = max(1, n // max_group_size)
  while num_groups % mesh_dim_size != 0 or n % num_groups != 0:
    num_groups += 1
  return num_groups, n // num_groups


def _expert_capacity(group_size, capacity_factor, num_experts, min_capacity):
  """Slots per expert per group (moe.py:368-371)."""
  capacity = min(group_size, int((group_size * capacity_factor) / num_experts))
  return max(capacity, min_capacity)


def _activation_names(activation):
  """mtf.relu / "relu" / None / "linear", or a list of those (the factors of
  mtf.layers.dense_product, layers.py:279-295) -> names understood by the
  kernels, one per factor."""
  if not isinstance(activation, (list, tuple)):
    activation = [activation]
  if not activation:
    raise ValueError("empty list of expert activations")
  names = []
  for a in activation:
    if a is None or a == "linear":
      names.append("linear")
      continue
    name = a if isinstance(a, str) else getattr(a, "__name__", None)
    if name not in moe_hip.ACTIVATIONS:
      raise NotImplementedError("expert activation %r is not implemented"
                                % (a,))
    names.append(name)
  return names


def _check_gating(hparams):
  if hparams.moe_gating in ("top_2", "switch", "switch_max", "ntlb",
                            "expert_selection"):
    return
  if hparams.moe_gating in _OTHER_GATINGS:
    raise NotImplementedError(
        "moe_gating=%s is not implemented"
        % hparams.moe_gating)
  raise ValueError("unknown hparams.moe_gating=%s" % hparams.moe_gating)


def _second_policy(hparams, train):
  if train:
    policy = hparams.moe_second_policy_train
    threshold = hparams.moe_second_threshold_train
  else:
    policy = hparams.moe_second_policy_eval
    threshold = hparams.moe_second_threshold_eval
  if policy not in moe_hip.POLICIES:
    raise ValueError("Unknown policy %s" % policy)
  return policy, threshold


class _GatingSpec(object):
  """Static configuration of one _top_2_gating call (moe.py:1312-1513)."""

  def __init__(self, hparams, train, num_microbatches):
    self.policy, self.threshold = _second_policy(hparams, train)
    self.use_second_place_loss = bool(hparams.moe_use_second_place_loss)
    self.num_microbatches = num_microbatches

  router = "top_2"
  z_loss = None
  summaries = False        # _top_2_gating emits no summaries

  def route(self, x, w, w_packed, group_size, num_experts, capacity,
            importance=None, importance_from_slot_gate=False,
            want_logits=False):
    """Router projection + gating of x [B, T, M] with routers w [B, M, E]
    (w_packed [B, E, M]); the B*T tokens form groups of group_size.  One fused
    launch sequence where the library has a kernel for the case, otherwise the
    projection and the gating as two calls.  Returns the Routing, and the
    float32 logits [G, S, E] too if want_logits."""
    b, t, _ = x.shape
    groups = b * t // group_size
    if moe_hip.fused_gating_supported(x, num_experts, group_size):
      uniform = None
      if self.policy == "random":
        uniform = torch.rand((groups, group_size), dtype=torch.float32,
                             device=x.device)
      return moe_hip.router_top2_gating(
          x, w_packed, group_size, capacity, importance=importance,
          policy=self.policy, threshold=self.threshold,
          use_second_place_loss=self.use_second_place_loss,
          num_microbatches=self.num_microbatches, second_uniform=uniform,
          importance_from_slot_gate=importance_from_slot_gate,
          want_logits=want_logits)
    logits = moe_hip.router_logits(x, w, w_packed=w_packed)
    logits = logits.reshape(groups, group_size, num_experts)
    r = self.run(logits, capacity, importance, importance_from_slot_gate)
    return (r, logits) if want_logits else r

  def run(self, logits, capacity, importance=None,
          importance_from_slot_gate=False):
    uniform = None
    if self.policy == "random":
      uniform = torch.rand(logits.shape[:2], dtype=torch.float32,
                           device=logits.device)
    return moe_hip.top2_gating(
        logits, capacity, importance=importance, policy=self.policy,
        threshold=self.threshold,
        use_second_place_loss=self.use_second_place_loss,
        num_microbatches=self.num_microbatches, second_uniform=uniform,
        importance_from_slot_gate=importance_from_slot_gate)


class _GateInputNoise(object):
  """The random multiplier the switch-family routers put on their input while
  training (hparams.moe_switch_policy_train):

  "input_jitter": u in [1 - eps, 1 + eps), eps = moe_switch_jitter
  (mtf.layers.multiplicative_jitter, layers.py:1949-1952);
  "input_dropout": (u < keep_prob) / keep_prob with keep_prob = 1 -
  moe_switch_dropout (mtf.dropout, ops.py:5864-5872).
  _switch_gating and _expert_selection_gating apply it to to_float(inputs)
  (moe.py:1189-1199, :1071-1078); _ntlb_gating knows only the jitter and
  applies it in the activation dtype (moe.py:821-822).  Only the router sees
  the perturbed tokens.  The uniform numbers come from torch's generator on the
  device (the reference's come from TensorFlow's)."""

  def __init__(self, hparams, train, in_float32, allow_dropout=True):
    policy = (hparams.moe_switch_policy_train if train
              else hparams.moe_switch_policy_eval)
    self.kind = None
    if train and policy == "input_jitter" and hparams.moe_switch_jitter != 0:
      self.kind = "jitter"
      self.eps = float(hparams.moe_switch_jitter)
    elif train and policy == "input_dropout" and allow_dropout and (
        hparams.moe_switch_dropout != 0):
      self.kind = "dropout"
      self.keep = 1.0 - float(hparams.moe_switch_dropout)
    self.in_float32 = in_float32
    self.last = None          # (router input, multiplier) of the last step

  def apply(self, x):
    """x [B, T, M] -> the router's input (float32 or x's dtype)."""
    self.last = None
    if self.kind is None:
      return x
    u = torch.rand(x.shape, dtype=torch.float32, device=x.device)
    if self.kind == "jitter":
      mult = (1.0 - self.eps) + u * (2.0 * self.eps)
    else:
      mult = (u < self.keep).to(torch.float32) / self.keep
    if self.in_float32:
      x_gate = x.to(torch.float32) * mult
    else:
      mult = mult.to(x.dtype)
      x_gate = x * mult
    self.last = (x_gate, mult)
    return x_gate


def _router_logits(x_gate, w, w_packed):
  """Router projection of a possibly float32 (perturbed) input with kernels of
  the activation dtype: the kernels are cast up, no packed copy is used."""
  if x_gate.dtype == w.dtype:
    return moe_hip.router_logits(x_gate, w, w_packed=w_packed)
  return moe_hip.router_logits(x_gate.contiguous(), w.to(x_gate.dtype))


class _SwitchGatingSpec(object):
  """Static configuration of one _switch_gating (moe.py:1176-1309) or
  _switch_max_gating (moe.py:943-1054) call: policies "argmax", "sample",
  "input_dropout" and "input_jitter" (the perturbations apply while training,
  moe.py:1192-1199)."""

  def __init__(self, hparams, train, num_microbatches, has_importance):
    self.slots_by_gate = hparams.moe_gating == "switch_max"
    policy = (hparams.moe_switch_policy_train if train
              else hparams.moe_switch_policy_eval)
    if policy not in ("argmax", "input_dropout", "input_jitter", "sample"):
      raise ValueError("Unknown Switch gating policy %s" % policy)
    # policy "sample" (moe.py:1213-1216): temperature 0 is the arg-max
    self.temperature = (float(hparams.moe_switch_temperature)
                        if policy == "sample" else 0.0)
    self.noise = _GateInputNoise(hparams, train, in_float32=True)
    self.z_loss = None                     # _switch_max_gating has no z-loss
    if (train and not self.slots_by_gate and
        getattr(hparams, "moe_z_loss", None) is not None):
      # the reference evaluates equal(importance, 1.0) and
      # denom * num_microbatches unconditionally (moe.py:1260-1264)
      if not has_importance or not num_microbatches:
        raise ValueError("moe_z_loss needs nonpadding and num_microbatches")
      self.z_loss = float(hparams.moe_z_loss)
    self.num_microbatches = num_microbatches
    # what the reference logs with mtf.scalar_summary while training
    # (moe.py:1213, :1242-1257, :1269, :1285-1289; :981, :1010-1025, :1041-1046)
    self.summaries = bool(train)
    self.summary_name = ("switch_max_gating" if self.slots_by_gate
                         else "switch_gating")
    self.logs_expert_gate = policy != "sample"

  router = "switch"
  use_second_place_loss = False

  def route(self, x, w, w_packed, group_size, num_experts, capacity,
            importance=None, importance_from_slot_gate=False,
            want_logits=False):
    """Same contract as _GatingSpec.route."""
    assert not importance_from_slot_gate
    b, t, _ = x.shape
    groups = b * t // group_size
    x_gate = self.noise.apply(x)
    if (x_gate is x and self.temperature == 0.0 and
        moe_hip.fused_gating_supported(x, num_experts, group_size)):
      return moe_hip.router_switch_gating(
          x, w_packed, group_size, capacity, importance=importance,
          z_loss=self.z_loss, num_microbatches=self.num_microbatches,
          slots_by_gate=self.slots_by_gate, want_logits=want_logits)
    logits = _router_logits(x_gate, w, w_packed)
    logits = logits.reshape(groups, group_size, num_experts)
    choice = None
    if self.temperature != 0.0:
      # mtf.sample_with_temperature (ops.py:5070-5086): Gumbel noise from
      # u in [1e-9, 1), arg-max of logits + noise * temperature
      u = torch.rand(logits.shape, dtype=torch.float32, device=logits.device)
      u = 1e-9 + u * (1.0 - 1e-9)
      choice = logits + (-torch.log(-torch.log(u))) * self.temperature
    r = moe_hip.switch_gating(
        logits, capacity, importance=importance, z_loss=self.z_loss,
        num_microbatches=self.num_microbatches,
        slots_by_gate=self.slots_by_gate, choice_logits=choice)
    return (r, logits) if want_logits else r


class _NtlbGatingSpec(object):
  """Static configuration of one _ntlb_gating call (moe.py:804-940); the only
  policy it knows is "input_jitter" while training."""

  router = "ntlb"
  use_second_place_loss = False
  z_loss = None

  def __init__(self, hparams, train, num_microbatches, has_importance):
    policy = (hparams.moe_switch_policy_train if train
              else hparams.moe_switch_policy_eval)
    del policy                                          # moe.py:816-822
    self.noise = _GateInputNoise(hparams, train, in_float32=False,
                                 allow_dropout=False)
    self.top_k = int(hparams.moe_ntlb_top_k)
    self.num_microbatches = num_microbatches
    self.summaries = bool(train)                        # moe.py:864-880
    self.summary_name = "ntlb_gating"

  def route(self, x, w, w_packed, group_size, num_experts, capacity,
            importance=None, importance_from_slot_gate=False,
            want_logits=False):
    """Same contract as _GatingSpec.route."""
    assert not importance_from_slot_gate
    b, t, _ = x.shape
    groups = b * t // group_size
    logits = _router_logits(self.noise.apply(x), w, w_packed)
    logits = logits.reshape(groups, group_size, num_experts)
    # the one router whose projection and softmax stay in the activation
    # dtype (moe.py:825-836)
    r = moe_hip.ntlb_gating(logits, capacity, self.top_k,
                            importance=importance,
                            num_microbatches=self.num_microbatches,
                            softmax_dtype=x.dtype)
    return (r, logits) if want_logits else r


class _ExpertSelectionGatingSpec(object):
  """Static configuration of one _expert_selection_gating call
  (moe.py:1057-1173): experts choose tokens.  The routing record is per slot
  (moe_hip.SlotRouting), so the layer dispatches and combines by slot."""

  router = "expert_selection"
  use_second_place_loss = False
  z_loss = None

  def __init__(self, hparams, train, num_microbatches, has_importance):
    policy = (hparams.moe_switch_policy_train if train
              else hparams.moe_switch_policy_eval)
    del policy                                          # moe.py:1064-1078
    self.noise = _GateInputNoise(hparams, train, in_float32=True)
    if not has_importance:
      # the reference sums `importance` for its loss (moe.py:1138-1140)
      raise ValueError("expert_selection gating needs nonpadding")
    self.num_microbatches = num_microbatches
    self.summaries = bool(train)                        # moe.py:1148-1165
    self.summary_name = "expert_selection_gating"

  def route(self, x, w, w_packed, group_size, num_experts, capacity,
            importance=None, importance_from_slot_gate=False,
            want_logits=False):
    assert not importance_from_slot_gate
    b, t, _ = x.shape
    groups = b * t // group_size
    logits = _router_logits(self.noise.apply(x), w, w_packed)
    logits = logits.reshape(groups, group_size, num_experts)
    r = moe_hip.expert_choice_gating(
        logits, capacity, importance=importance,
        num_microbatches=self.num_microbatches)
    return (r, logits) if want_logits else r


def _emit_router_summaries(lowering, spec, logits, r, capacity, importance,
                           act_dtype, scope):
  """The scalar summaries the f1 routers log while training, computed by
  mesh_moe_router_summaries from the router's logits and record and recorded
  on the Lowering under the reference's names.  The per-expert (per group
  position) names follow "experts/" + fraction.name.replace(":", "/")
  (moe.py:877-879): the outputs of an mtf.split named "split" in the layer's
  scope."""
  by_slot = isinstance(r, moe_hip.SlotRouting)
  vals = moe_hip.router_summaries(
      logits, spec.router if not getattr(spec, "slots_by_gate", False)
      else "switch_max", capacity, importance=importance,
      kept=None if by_slot else r.kept,
      tok_slot=r.tok_slot if by_slot else None,
      top_k=getattr(spec, "top_k", 1),
      num_microbatches=spec.num_microbatches,
      softmax_dtype=act_dtype if spec.router == "ntlb" else torch.float32)
  add = lowering.add_scalar_summary
  aux_loss = r.loss[0]
  if spec.router == "switch" and getattr(spec, "logs_expert_gate", False):
    add("expert_gate", vals[1])
  add(spec.summary_name + "/entropy", vals[0])
  prefix = ("group_token/" if by_slot else "experts/") + (
      scope + "/" if scope else "")
  for i in range(vals.shape[0] - 4):
    add("%ssplit/%d" % (prefix, i), vals[4 + i])
  if spec.z_loss is not None:
    aux_loss = aux_loss - spec.z_loss * vals[3]
  add("aux_loss", aux_loss)
  if spec.z_loss is not None:
    add(spec.summary_name + "/z_loss", vals[3])
  if spec.router == "switch":
    add("fraction_routed", vals[2])


def _packed(lowering, kernel_tensor, dtype):
  """K-contiguous copy of an expert kernel variable, cached on the variable."""
  return lowering.variables[kernel_tensor.operation].packed(dtype)


def _release_saved(saved):
  """Called by a gradient operation when it has run: the activations the
  forward operation kept for it (several GiB at the largest benchmark layer)
  are dropped once the last gradient operation built on that forward
  operation has consumed them, instead of living until the next step."""
  saved["_consumers"] = saved.get("_consumers", 1) - 1
  if saved["_consumers"] <= 0:
    saved.clear()


class MoEV1Operation(mtf.Operation):
  """The whole of transformer_moe_layer_v1 after the reshape to groups:
  inputs [outer_batch, groups, group, d_model] -> (outputs with d_model
  replaced by output_dim, scalar balancing loss before moe_loss_coef)."""

  def __init__(self, inputs, w_gate, wi, wo, importance, output_dim, capacity,
               gating, activation, k_wo=None, hidden_keep_prob=None,
               name="moe_v1"):
    """With k_wo (moe_use_experts_attention, moe.py:514-522) `wo` is the "q_wo"
    kernel, the operation has a second output projection of the same hidden
    tensor and its outputs are (q, loss, k).

    `wi` and `activation` may be lists of the same length: the hidden tensor
    is then the product of act_i(expert_in . wi_i) (moe.py:469-475).
    hidden_keep_prob: keep probability of the dropout on the hidden tensor
    (moe.py:477-479), None for none."""
    wis = list(wi) if isinstance(wi, (list, tuple)) else [wi]
    acts = (list(activation) if isinstance(activation, (list, tuple))
            else [activation])
    if len(wis) != len(acts):
      raise ValueError("%d wi kernels for %d activations"
                       % (len(wis), len(acts)))
    wi = wis[0]
    ins = [inputs, w_gate, wi, wo] + ([importance] if importance is not None
                                      else [])
    if k_wo is not None:
      ins.append(k_wo)
    ins.extend(wis[1:])
    super(MoEV1Operation, self).__init__(ins, name=name)
    self._scope = mtf.current_scope_name()
    self._has_importance = importance is not None
    self._k_wo = k_wo
    self._capacity = capacity
    self._gating = gating
    self._activation = acts[0]
    self._more_wi = wis[1:]
    self._more_activations = acts[1:]
    self._hidden_keep_prob = hidden_keep_prob
    # experts that are not one ReLU / linear layer: the backward pass needs the
    # pre-activation of every factor
    self._general_hidden = bool(self._more_wi) or (
        self._activation not in ("relu", "linear"))
    self._num_experts = wi.shape.dims[0].size
    self._save_for_backward = False
    out_shape = mtf.Shape(inputs.shape.dims[:-1] + [output_dim])
    self._outputs = [mtf.Tensor(self, out_shape, inputs.dtype, index=0),
                     mtf.Tensor(self, mtf.Shape([]), inputs.dtype, index=1)]
    if k_wo is not None:
      self._outputs.append(mtf.Tensor(self, out_shape, inputs.dtype, index=2))

  def gradient(self, grad_ys):
    """Gradients w.r.t. (inputs, gate kernel, wi, wo[, importance][, k_wo])
    from those of (outputs, loss[, second outputs]); importance carries
    none."""
    self._save_for_backward = True
    self._num_grad_ops = getattr(self, "_num_grad_ops", 0) + 1
    d_out, d_loss = grad_ys[:2]
    if d_out is None:
      d_out = mtf.zeros(self.mesh, self.outputs[0].shape, self.outputs[0].dtype)
    if d_loss is None:
      d_loss = mtf.zeros(self.mesh, mtf.Shape([]), self.outputs[1].dtype)
    d_k = None
    if self._k_wo is not None:
      d_k = grad_ys[2]
      if d_k is None:
        d_k = mtf.zeros(self.mesh, self.outputs[2].shape, self.outputs[2].dtype)
    grad_op = MoEV1GradOperation(self, d_out, d_loss, d_k)
    by_input = dict(zip(grad_op.wrt, grad_op.outputs))
    return [by_input.get(t) for t in self.inputs]

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    x, w_gate, wi, wo = self.inputs[:4]
    dt = x.dtype
    wi_p = _packed(lowering, wi, dt)
    wo_p = _packed(lowering, wo, dt)
    wg_p = _packed(lowering, w_gate, dt)               # [1, E, M]
    kwo_p = (_packed(lowering, self._k_wo, dt) if self._k_wo is not None
             else None)
    more_wi_p = [_packed(lowering, t, dt) for t in self._more_wi]
    keep_prob = self._hidden_keep_prob
    keep_pre = self._save_for_backward and self._general_hidden
    plain_hidden = not more_wi_p and keep_prob is None and not keep_pre
    o_, g_, s_, m_ = x.shape.to_integer_list
    n_ = self.outputs[0].shape.dims[-1].size
    e_, c_ = self._num_experts, self._capacity
    groups = o_ * g_

    save = self._save_for_backward
    saved = {}

    def fn(x_s, wg_s, imp_s=None):
      xg = x_s.reshape(groups, s_, m_)
      if imp_s is not None:
        imp_s = imp_s.reshape(groups, s_)
      summarize = self._gating.summaries
      r = self._gating.route(xg.reshape(1, groups * s_, m_),
                             wg_s.reshape(1, m_, e_), wg_p, s_, e_, c_, imp_s,
                             want_logits=save or summarize)
      logits = None
      if save or summarize:
        r, logits = r
      if summarize:
        _emit_router_summaries(lowering, self._gating, logits, r, c_, imp_s, dt,
                               self._scope)
        if not save:
          logits = None
      by_slot = isinstance(r, moe_hip.SlotRouting)
      y = None
      noise = None
      row_offsets = None
      expert_in = h = None
      # one relu / linear / ... layer per expert, with or without the hidden
      # dropout: what the compacted calls take
      one_layer = not more_wi_p and not keep_pre
      single_choice = (not by_slot and kwo_p is None and one_layer and
                       self._gating.router != "top_2")
      # Top-2 also runs on compacted rows where an expert's slot rows are
      # whole 256-row tiles (no tile is saved, the empty slots only move to
      # the end of each expert's rows; measured 1.5 % faster forward and 1 %
      # forward + backward at 64 experts x 2048 slots, d_model 4096, d_ff
      # 16384).  Other row counts keep the padded layout, whose last row tile
      # per expert is shortened instead.
      compact_forward = single_choice or (
          not by_slot and kwo_p is None and one_layer and
          (groups * c_) % 256 == 0)

      # the gradient of ReLU experts takes the dropout's noise from the stored
      # activation (positive = kept, 1 / keep_prob there): no noise tensor
      keep_noise = save and (self._general_hidden or self._activation != "relu")

      def compact_ffn(want_hidden):
        """The expert feed-forward on compacted rows (the occupied slots at
        the front of every expert's rows), hidden dropout included; None where
        the library has no such kernel for the case."""
        u = None
        if keep_prob is not None:
          u = torch.rand((e_, groups * c_, wi_p.shape[1]), dtype=dt,
                         device=xg.device)
        return moe_hip.compact_expert_ffn(
            xg, r, wi_p, wo_p, self._activation, want_hidden=want_hidden,
            uniform=u, keep_prob=1.0 if keep_prob is None else keep_prob,
            want_noise=want_hidden and keep_noise)

      if (save and compact_forward and
          moe_hip.compact_training_applies(xg, r, wi_p.shape[1], n_,
                                           self._activation)):
        # a gradient to follow: the occupied slots at the front of every
        # expert's rows in all the tensors the gradient operation reads, so
        # that it too multiplies only those
        compact = compact_ffn(True)
        if compact is not None:
          y, row_offsets, h = compact[:3]
          noise = compact[3] if len(compact) > 3 else None
          expert_in = moe_hip.dispatch(xg, r, row_offsets=row_offsets)
          expert_in = expert_in.reshape(e_, groups * c_, m_)
      if not save and compact_forward:
        # Routers with one choice per token leave about 1 - 1 / capacity_factor
        # of the slots empty: their occupied slots are moved to the front of
        # every expert's rows and only the tiles that hold them are multiplied
        compact = compact_ffn(False)
        if compact is not None:
          y, row_offsets = compact
      if (y is None and not (save or by_slot or kwo_p is not None) and
          plain_hidden):
        # nobody reads expert_in afterwards: fold the dispatch into the first
        # expert GEMM where the library can
        y = moe_hip.dispatched_expert_ffn(xg, r, wi_p, wo_p,
                                          self._activation)
      if y is None:
        expert_in = (moe_hip.slot_dispatch(xg, r) if by_slot
                     else moe_hip.dispatch(xg, r))
        expert_in = expert_in.reshape(e_, groups * c_, m_)
      if y is None and plain_hidden:
        h = None
        if save or kwo_p is not None:
          h = torch.empty((e_, groups * c_, wi_p.shape[1]), dtype=dt,
                          device=xg.device)
        y = moe_hip.expert_ffn(expert_in, wi_p, wo_p, self._activation, h=h)
      elif y is None:
        # the hidden tensor is worked on between the two projections: the
        # other factors of the product, then the dropout
        pres, factors = [], []
        for w_p, act in zip([wi_p] + more_wi_p,
                            [self._activation] + self._more_activations):
          if keep_pre:
            pres.append(moe_hip.expert_linear(expert_in, w_p, "linear"))
            factors.append(moe_hip.activation(pres[-1], act))
          else:
            factors.append(moe_hip.expert_linear(expert_in, w_p, act))
        h = factors[0].clone() if (keep_pre and len(factors) > 1) else factors[0]
        for f in factors[1:]:
          moe_hip.hidden_product(h, factor=f)
        if keep_pre:
          if len(factors) == 1 and keep_prob is not None:
            factors[0] = None       # h is about to be changed in place
          saved.update(pre=pres, factors=factors)
        if keep_prob is not None:
          u = torch.rand(h.shape, dtype=dt, device=h.device)
          noise = moe_hip.hidden_product(h, uniform=u, keep_prob=keep_prob,
                                         want_noise=keep_noise)
        y = moe_hip.expert_linear(h, wo_p)
      y4 = y.reshape(e_, groups, c_, n_)
      out = (moe_hip.slot_combine(y4, r, s_) if by_slot
             else moe_hip.combine(y4, r, s_, row_offsets=row_offsets))
      if save:
        # what the gradient operation reads (activations of this step)
        gate_noise = getattr(self._gating, "noise", None)
        gate_in = gate_noise.last if gate_noise is not None else None
        saved.update(x=xg, routing=r, logits=logits, importance=imp_s,
                     expert_in=expert_in, h=h, y=y, row_offsets=row_offsets,
                     w_gate_packed=wg_p,
                     gate_in=gate_in, w_gate=wg_s, hidden_noise=noise)
      outs = (out.reshape(o_, g_, s_, n_), r.loss.to(dt).reshape(()))
      if kwo_p is not None:
        # the "k" projection of the same hidden tensor (moe.py:514-520)
        yk = moe_hip.expert_linear(h, kwo_p).reshape(e_, groups, c_, n_)
        if save:
          saved.update(yk=yk)
        out_k = (moe_hip.slot_combine(yk, r, s_) if by_slot
                 else moe_hip.combine(yk, r, s_))
        outs = outs + (out_k.reshape(o_, g_, s_, n_),)
      return outs

    args = [lowering.tensors[x], lowering.tensors[w_gate]]
    if self._has_importance:
      args.append(lowering.tensors[self.inputs[4]])
    outs = mesh_impl.slicewise(fn, *args)
    for t, v in zip(self.outputs, outs):
      lowering.set_tensor_lowering(t, v)
    if saved:
      saved["_consumers"] = getattr(self, "_num_grad_ops", 0)
    lowering.operations[self] = saved


class MoEV1GradOperation(mtf.Operation):
  """Backward of MoEV1Operation: (d outputs, d loss) -> gradients of the
  tokens and of the three kernels, in the activation dtype.

  The reference gets these from mtf.gradients over the layer's einsums
  (mesh_tensorflow/ops.py:5254-5291, :2846-2854); here they are one call
  sequence into the HIP library on the activations the forward operation
  kept."""

  def __init__(self, forward, d_out, d_loss, d_k=None, name="moe_v1_grad"):
    """d_k: gradient of the second outputs of a layer with
    moe_use_experts_attention; the operation then has a fifth output, the
    gradient of the "k_wo" kernel."""
    ins = forward.inputs[:4] + [d_out, d_loss]
    wrt = forward.inputs[:4]
    if d_k is not None:
      ins = ins + [forward._k_wo, d_k]
      wrt = wrt + [forward._k_wo]
    # the kernels of the other factors of a product of dense layers
    ins = ins + forward._more_wi
    wrt = wrt + forward._more_wi
    super(MoEV1GradOperation, self).__init__(ins, name=name)
    self._forward = forward
    self._has_k = d_k is not None
    self.wrt = wrt          # the tensors the outputs are gradients of
    self._outputs = [mtf.Tensor(self, t.shape, t.dtype, index=i)
                     for i, t in enumerate(wrt)]

  @property
  def has_gradient(self):
    return False

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    fwd = self._forward
    x, w_gate, wi, wo = fwd.inputs[:4]
    o_, g_, s_, m_ = x.shape.to_integer_list
    e_, c_ = fwd._num_experts, fwd._capacity
    n_ = fwd.outputs[0].shape.dims[-1].size
    groups = o_ * g_
    gating = fwd._gating

    has_k, n_more = self._has_k, len(fwd._more_wi)
    activations = [fwd._activation] + fwd._more_activations

    def general_hidden_backward(sv, dys, wos, wis):
      """Experts that are not one ReLU / linear layer: h = noise * prod_i
      act_i(expert_in . wi_i).  dys / wos: the gradient and the kernel of every
      output projection of h.  Returns (dexpert_in, [dwi_i], [dwo_j])."""
      xe = sv["expert_in"].reshape(e_, groups * c_, m_)
      dh, dwos = None, []
      for dy_j, wo_j in zip(dys, wos):
        dh_j, dwo_j = moe_hip.expert_linear_backward(sv["h"], dy_j, wo_j)
        dh = dh_j if dh is None else dh + dh_j
        dwos.append(dwo_j)
      if sv["hidden_noise"] is not None:
        moe_hip.hidden_product(dh, factor=sv["hidden_noise"])
      dxe, dwis = None, []
      for i, act in enumerate(activations):
        g = dh
        for j, f in enumerate(sv["factors"]):
          if j != i:
            g = g.clone() if g is dh else g
            moe_hip.hidden_product(g, factor=f)
        dpre = moe_hip.activation_backward(g, sv["pre"][i], act)
        dxe_i, dwi_i = moe_hip.expert_linear_backward(xe, dpre, wis[i])
        dxe = dxe_i if dxe is None else dxe + dxe_i
        dwis.append(dwi_i)
      return dxe, dwis, dwos

    def fn(wi_s, wo_s, dout_s, dloss_s, *rest):
      kwo_s, dk_s = rest[:2] if has_k else (None, None)
      more_wi_s = list(rest[2 if has_k else 0:])
      sv = lowering.operations[fwd]
      if not sv:
        raise ValueError("the forward operation kept no activations: build "
                         "the gradient before lowering the graph")
      r = sv["routing"]
      by_slot = isinstance(r, moe_hip.SlotRouting)
      combine_backward = (moe_hip.slot_combine_backward if by_slot
                          else moe_hip.combine_backward)
      # the forward pass may have put the occupied slots first in every
      # tensor with slot rows
      row_offsets = sv.get("row_offsets")
      compact = {} if row_offsets is None else {"row_offsets": row_offsets}
      dy, dgate = combine_backward(
          dout_s.reshape(groups, s_, n_).contiguous(),
          sv["y"].reshape(e_, groups, c_, n_), r, **compact)
      if row_offsets is not None:
        dxe, dwi, dwo = moe_hip.compact_expert_ffn_backward(
            sv["expert_in"].reshape(e_, groups * c_, m_), sv["h"],
            dy.reshape(e_, groups * c_, n_), wi_s, wo_s, r, row_offsets,
            fwd._activation, dh_scale=sv["hidden_noise"],
            keep_prob=fwd._hidden_keep_prob)
        dkwo, dwis = None, [dwi]
      elif fwd._general_hidden:
        dys, wos = [dy.reshape(e_, groups * c_, n_)], [wo_s]
        if has_k:
          dyk, dgate_k = combine_backward(
              dk_s.reshape(groups, s_, n_).contiguous(),
              sv["yk"].reshape(e_, groups, c_, n_), r)
          dys.append(dyk.reshape(e_, groups * c_, n_))
          wos.append(kwo_s)
          dgate = dgate + dgate_k
        dxe, dwis, dwos = general_hidden_backward(sv, dys, wos,
                                                  [wi_s] + more_wi_s)
        dwi, dwo = dwis[0], dwos[0]
        dkwo = dwos[1] if has_k else None
        kwo_s = None                        # its share is in already
      else:
        dxe, dwi, dwo = moe_hip.expert_ffn_backward(
            sv["expert_in"].reshape(e_, groups * c_, m_), sv["h"],
            dy.reshape(e_, groups * c_, n_), wi_s, wo_s, fwd._activation,
            dh_scale=sv["hidden_noise"],
            keep_prob=fwd._hidden_keep_prob)
        dkwo, dwis = None, [dwi]
      if kwo_s is not None:
        # the second projection of the same hidden tensor: its share of every
        # gradient adds to the first one's (the hidden tensor and the combine
        # weights have two consumers)
        dyk, dgate_k = combine_backward(
            dk_s.reshape(groups, s_, n_).contiguous(),
            sv["yk"].reshape(e_, groups, c_, n_), r)
        dxe_k, dwi_k, dkwo = moe_hip.expert_ffn_backward(
            sv["expert_in"].reshape(e_, groups * c_, m_), sv["h"],
            dyk.reshape(e_, groups * c_, n_), wi_s, kwo_s, fwd._activation,
            dh_scale=sv["hidden_noise"],
            keep_prob=fwd._hidden_keep_prob)
        dxe, dwi, dgate = dxe + dxe_k, dwi + dwi_k, dgate + dgate_k
      if by_slot:
        dlogits = moe_hip.expert_choice_backward(
            sv["logits"], r, dgate, dloss_s.reshape(1).float(), 1.0,
            importance=sv["importance"],
            num_microbatches=gating.num_microbatches)
        dispatch_backward = moe_hip.slot_dispatch_backward
      else:
        dlogits = moe_hip.gating_backward(
            sv["logits"], r, dgate, dloss_s.reshape(1).float(), 1.0,
            router=gating.router, top_k=getattr(gating, "top_k", 0),
            importance=sv["importance"], z_loss=gating.z_loss,
            num_microbatches=gating.num_microbatches,
            use_second_place_loss=gating.use_second_place_loss,
            softmax_dtype=(sv["x"].dtype if gating.router == "ntlb"
                           else torch.float32))
        dispatch_backward = moe_hip.dispatch_backward
      tokens = groups * s_
      if sv["gate_in"] is None:
        dwg = moe_hip.router_backward_weights(
            sv["x"].reshape(tokens, m_), dlogits.reshape(tokens, e_))
        # the router kernel as the variable holds it, [M, E]
        compact = dict(compact, w_gate=sv["w_gate"].reshape(m_, e_).to(
            sv["x"].dtype).contiguous())
        dx = dispatch_backward(
            dxe.reshape(e_, groups, c_, m_), r, s_, dlogits,
            sv["w_gate_packed"].reshape(e_, m_), **compact)
      else:
        # the router saw x * mult (a constant of the graph): its kernel's
        # gradient uses that input, and its share of d(tokens) is
        # (dlogits . w_gate^T) * mult
        x_gate, mult = sv["gate_in"]
        dt = sv["x"].dtype
        dwg = moe_hip.router_backward_weights(
            x_gate.reshape(tokens, m_).contiguous(),
            dlogits.reshape(tokens, e_)).to(dt)
        dx = dispatch_backward(dxe.reshape(e_, groups, c_, m_), r, s_,
                               **compact)
        w32 = sv["w_gate"].reshape(1, m_, e_).to(torch.float32).contiguous()
        dx_router = moe_hip.expert_linear(
            dlogits.reshape(1, tokens, e_), w32, "linear")   # [1, T, M]
        dx = (dx.reshape(tokens, m_).to(torch.float32) +
              dx_router.reshape(tokens, m_) *
              mult.reshape(tokens, m_).to(torch.float32)).to(dt)
      res = (dx.reshape(o_, g_, s_, m_), dwg, dwi, dwo)
      if has_k:
        res = res + (dkwo,)
      return res + tuple(dwis[1:])

    ins = self.inputs
    args = [lowering.tensors[ins[i]] for i in (2, 3, 4, 5)]
    args += [lowering.tensors[t] for t in ins[6:]]
    outs = mesh_impl.slicewise(fn, *args)
    _release_saved(lowering.operations[fwd])
    for t, v in zip(self.outputs, outs):
      lowering.set_tensor_lowering(t, v)


def transformer_moe_layer_v1(
    inputs, output_dim, hparams, train, variable_dtype,
    layout=None, mesh_shape=None, nonpadding=None, activation=mtf.relu,
    num_microbatches=None):
  """Local mixture of experts: each position goes to 0-2 experts chosen by a
  learned top-2 gate (moe_gating="top_2") or to 0-1 experts chosen by a switch
  gate (moe_gating="switch"), with a fixed per-group capacity per expert.

  Args:
    inputs: a mtf.Tensor with shape [batch_dim(s), length_dim, input_dim]
    output_dim: a mtf.Dimension (for Transformer, this is input_dim)
    hparams: model hyperparameters (moe_num_experts, moe_hidden_size,
      moe_group_size, moe_capacity_factor_train/eval, moe_min_expert_capacity,
      moe_gating, moe_dropout_rate, moe_use_experts_attention, moe_loss_coef,
      moe_use_second_place_loss, moe_second_policy_train/eval,
      moe_second_threshold_train/eval; for switch gating
      moe_switch_policy_train/eval and moe_z_loss)
    train: a boolean
    variable_dtype: a mtf.VariableDType
    layout: optional - an input to mtf.convert_to_layout_rules
    mesh_shape: optional - an input to mtf.convert_to_shape
    nonpadding: an optional Tensor with shape [batch_dim(s), length_dim]
      and the same dtype as inputs, consisting of ones(nonpadding)
      and zeros(padding).
    activation: a function, or the name of one.
    num_microbatches: number of microbatches.

  Returns:
    outputs: a Tensor with shape [batch_dim(s), length_dim, output_dim]
    loss: a mtf scalar

  Raises:
    ValueError: on unrecognized hparams.moe_gating
  """
  orig_inputs = inputs
  hidden_dim = mtf.Dimension("expert_hidden", hparams.moe_hidden_size)
  experts_dim = mtf.Dimension("experts", hparams.moe_num_experts)
  batch_and_length_dims = orig_inputs.shape.dims[:-1]
  input_dim = orig_inputs.shape.dims[-1]
  if orig_inputs.shape.dims[0].name == "outer_batch":
    outer_batch_dim, orig_batch_dim = orig_inputs.shape.dims[:2]
  else:
    outer_batch_dim = mtf.Dimension("outer_batch", 1)
    orig_batch_dim = orig_inputs.shape.dims[0]

  n = mtf.list_product(d.size for d in batch_and_length_dims)
  n = n // outer_batch_dim.size
  mesh_dim_size = mtf.tensor_dim_to_mesh_dim_size(layout, mesh_shape,
                                                  orig_batch_dim)
  num_groups, group_size = _split_into_groups(n, hparams.moe_group_size,
                                              mesh_dim_size)
  group_size_dim = mtf.Dimension("group", group_size)
  num_groups_dim = mtf.Dimension(orig_batch_dim.name, num_groups)
  moe_input_dims = [outer_batch_dim, num_groups_dim, group_size_dim, input_dim]
  inputs = mtf.reshape(inputs, moe_input_dims)

  capacity_factor = (hparams.moe_capacity_factor_train if train
                     else hparams.moe_capacity_factor_eval)
  expert_capacity = _expert_capacity(group_size_dim.size, capacity_factor,
                                     experts_dim.size,
                                     hparams.moe_min_expert_capacity)
  experts_dim_unsplit = mtf.Dimension("expert_unsplit", experts_dim.size)
  if nonpadding is not None:
    nonpadding = mtf.zeros(
        inputs.mesh, batch_and_length_dims, dtype=inputs.dtype) + nonpadding
    nonpadding = mtf.reshape(nonpadding, moe_input_dims[:-1])

  _check_gating(hparams)
  hidden_keep_prob = None
  if hparams.moe_dropout_rate != 0.0 and train:
    hidden_keep_prob = 1.0 - hparams.moe_dropout_rate   # moe.py:477-479
  if hparams.moe_gating == "expert_selection":
    gating = _ExpertSelectionGatingSpec(hparams, train, num_microbatches,
                                        nonpadding is not None)
    router_name = "expert_selection_gating"             # moe.py:1061
  elif hparams.moe_gating in ("switch", "switch_max"):
    gating = _SwitchGatingSpec(hparams, train, num_microbatches,
                               nonpadding is not None)
    router_name = hparams.moe_gating + "_gating"        # moe.py:1178, :945
  elif hparams.moe_gating == "ntlb":
    gating = _NtlbGatingSpec(hparams, train, num_microbatches,
                             nonpadding is not None)
    router_name = "ntlb_gating"                         # moe.py:812
  else:
    gating = _GatingSpec(hparams, train, num_microbatches)
    router_name = "top_2_gating"                        # moe.py:1314
  act_names = _activation_names(activation)

  # variables, named and shaped as the reference's dense layers create them
  w_gate = mtf_layers.get_dense_kernel_weights(
      inputs, [experts_dim_unsplit], [input_dim], [], None,
      name=router_name, variable_dtype=variable_dtype)
  # one kernel per factor of the product, "wi" or "wi_0", "wi_1", ...
  # (layers.py:293)
  wi = [mtf_layers.get_dense_kernel_weights(
      inputs, [hidden_dim], [input_dim], [experts_dim], None,
      name="wi_%d" % i if len(act_names) > 1 else "wi",
      variable_dtype=variable_dtype) for i in range(len(act_names))]
  if hparams.moe_use_experts_attention:
    # two output projections of the same hidden tensor (moe.py:514-522)
    q_wo = mtf_layers.get_dense_kernel_weights(
        inputs, [output_dim], [hidden_dim], [experts_dim], None, name="q_wo",
        variable_dtype=variable_dtype)
    k_wo = mtf_layers.get_dense_kernel_weights(
        inputs, [output_dim], [hidden_dim], [experts_dim], None, name="k_wo",
        variable_dtype=variable_dtype)
    q, loss, k = MoEV1Operation(
        inputs, w_gate, wi, q_wo, nonpadding, output_dim, expert_capacity,
        gating, act_names, k_wo=k_wo,
        hidden_keep_prob=hidden_keep_prob).outputs
    outputs = [mtf.reshape(t, batch_and_length_dims + [output_dim])
               for t in (q, k)]
    return outputs, loss * hparams.moe_loss_coef
  wo = mtf_layers.get_dense_kernel_weights(
      inputs, [output_dim], [hidden_dim], [experts_dim], None, name="wo",
      variable_dtype=variable_dtype)

  output, loss = MoEV1Operation(
      inputs, w_gate, wi, wo, nonpadding, output_dim, expert_capacity, gating,
      act_names, hidden_keep_prob=hidden_keep_prob).outputs
  output = mtf.reshape(output, batch_and_length_dims + [output_dim])
  return output, loss * hparams.moe_loss_coef


class MoEV2Operation(mtf.Operation):
  """The whole of transformer_moe_layer_v2 after the reshape to groups:
  inputs [a0, g1, s, m] -> (outputs [a0, g1, s, n], loss_outer + loss_inner).

  Level 1 routes tokens to expert groups x with capacity c; the occupied slots
  of each x, taken in (a0, g, c) order, are regrouped into h0 groups of t and
  routed again to experts y with capacity d, with importance 1.0 for slots
  holding a first choice, 0.5 for a second choice and 0 for empty slots
  (moe.py:692-801)."""

  def __init__(self, inputs, w_outer, w_inner, wi, wo, importance, output_dim,
               dims, gating, name="moe_v2"):
    ins = [inputs, w_outer, w_inner, wi, wo] + (
        [importance] if importance is not None else [])
    super(MoEV2Operation, self).__init__(ins, name=name)
    self._has_importance = importance is not None
    self._dims = dims
    self._gating = gating
    self._save_for_backward = False
    out_shape = mtf.Shape(inputs.shape.dims[:-1] + [output_dim])
    self._outputs = [mtf.Tensor(self, out_shape, inputs.dtype, index=0),
                     mtf.Tensor(self, mtf.Shape([]), inputs.dtype, index=1)]

  def gradient(self, grad_ys):
    """Gradients w.r.t. (inputs, outer / inner gate kernels, wi, wo
    [, importance]) from those of (outputs, loss)."""
    self._save_for_backward = True
    self._num_grad_ops = getattr(self, "_num_grad_ops", 0) + 1
    d_out, d_loss = grad_ys
    if d_out is None:
      d_out = mtf.zeros(self.mesh, self.outputs[0].shape, self.outputs[0].dtype)
    if d_loss is None:
      d_loss = mtf.zeros(self.mesh, mtf.Shape([]), self.outputs[1].dtype)
    grads = MoEV2GradOperation(self, d_out, d_loss).outputs
    return grads + [None] * (len(self.inputs) - 5)

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    x, w_outer, w_inner, wi, wo = self.inputs[:5]
    dt = x.dtype
    wi_p = _packed(lowering, wi, dt)      # [y*x, hidden, m]
    wo_p = _packed(lowering, wo, dt)      # [y*x, n, hidden]
    w_outer_p = _packed(lowering, w_outer, dt)         # [1, x, m]
    w_inner_p = _packed(lowering, w_inner, dt)         # [x, y, m]
    a0, g1, s_, m_ = x.shape.to_integer_list
    n_ = self.outputs[0].shape.dims[-1].size
    x_e, y_e, c_, h0, t_, d_ = self._dims
    ag = a0 * g1

    save = self._save_for_backward
    saved = {}

    def fn(x_s, wo_s, wi_s, imp_s=None):
      xg = x_s.reshape(ag, s_, m_)
      # outer level
      if imp_s is not None:
        imp_s = imp_s.reshape(ag, s_)
      rx = self._gating.route(xg.reshape(1, ag * s_, m_),
                              wo_s.reshape(1, m_, x_e), w_outer_p, s_, x_e, c_,
                              imp_s, want_logits=save)
      logits_x = None
      if save:
        rx, logits_x = rx
      ein_x, slot_gate = moe_hip.dispatch(xg, rx, want_slot_gate=True)
      # inner level: each outer expert's a0*g*c slots become h0 groups of t
      inputs_y = ein_x.reshape(x_e, h0 * t_, m_)
      ry = self._gating.route(inputs_y, wi_s, w_inner_p, t_, y_e, d_,
                              slot_gate.reshape(x_e * h0, t_),
                              importance_from_slot_gate=True, want_logits=save)
      logits_y = None
      if save:
        ry, logits_y = ry
      ein_y = moe_hip.dispatch(inputs_y.reshape(x_e * h0, t_, m_), ry)
      # experts: weights are [y, x, ...]; rows of (y, x) are its h0*d slots
      h = None
      if save:
        h = torch.empty((y_e * x_e, h0 * d_, wi_p.shape[1]), dtype=dt,
                        device=xg.device)
      yy = moe_hip.expert_ffn(ein_y.reshape(y_e * x_e, h0 * d_, m_), wi_p,
                              wo_p, "relu", h=h)
      out_y = moe_hip.combine(yy.reshape(y_e, x_e * h0, d_, n_), ry, t_)
      out = moe_hip.combine(out_y.reshape(x_e, ag, c_, n_), rx, s_)
      loss = (rx.loss.to(dt) + ry.loss.to(dt)).reshape(())
      if save:
        saved.update(x=xg, rx=rx, ry=ry, logits_x=logits_x, logits_y=logits_y,
                     importance=imp_s, slot_gate=slot_gate, inputs_y=inputs_y,
                     ein_y=ein_y, h=h, yy=yy, out_y=out_y,
                     w_outer_packed=w_outer_p, w_inner_packed=w_inner_p,
                     w_outer=wo_s.reshape(1, m_, x_e).to(dt).contiguous(),
                     w_inner=wi_s.reshape(x_e, m_, y_e).to(dt).contiguous())
      return out.reshape(a0, g1, s_, n_), loss

    args = [lowering.tensors[x], lowering.tensors[w_outer],
            lowering.tensors[w_inner]]
    if self._has_importance:
      args.append(lowering.tensors[self.inputs[5]])
    out, loss = mesh_impl.slicewise(fn, *args)
    lowering.set_tensor_lowering(self.outputs[0], out)
    lowering.set_tensor_lowering(self.outputs[1], loss)
    if saved:
      saved["_consumers"] = getattr(self, "_num_grad_ops", 0)
    lowering.operations[self] = saved


class MoEV2GradOperation(mtf.Operation):
  """Backward of MoEV2Operation: the v1 call sequence twice, inner level first
  (combine outer, combine inner, experts, inner gating / router / dispatch,
  outer gating / router / dispatch).  The inner importance is a comparison of
  slot weights (moe.py:725-727) and carries no gradient."""

  def __init__(self, forward, d_out, d_loss, name="moe_v2_grad"):
    super(MoEV2GradOperation, self).__init__(
        forward.inputs[:5] + [d_out, d_loss], name=name)
    self._forward = forward
    self._outputs = [mtf.Tensor(self, t.shape, t.dtype, index=i)
                     for i, t in enumerate(forward.inputs[:5])]

  @property
  def has_gradient(self):
    return False

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    fwd = self._forward
    x = fwd.inputs[0]
    a0, g1, s_, m_ = x.shape.to_integer_list
    n_ = fwd.outputs[0].shape.dims[-1].size
    x_e, y_e, c_, h0, t_, d_ = fwd._dims
    ag = a0 * g1
    gating = fwd._gating

    def fn(wi_s, wo_s, dout_s, dloss_s):
      sv = lowering.operations[fwd]
      if not sv:
        raise ValueError("the forward operation kept no activations: build "
                         "the gradient before lowering the graph")
      rx, ry = sv["rx"], sv["ry"]
      dl = dloss_s.reshape(1).float()
      hdim = wi_s.shape[-1]
      d_eo_x, dgate_x = moe_hip.combine_backward(
          dout_s.reshape(ag, s_, n_).contiguous(),
          sv["out_y"].reshape(x_e, ag, c_, n_), rx)
      dyy, dgate_y = moe_hip.combine_backward(
          d_eo_x.reshape(x_e * h0, t_, n_),
          sv["yy"].reshape(y_e, x_e * h0, d_, n_), ry)
      dein_y, dwi, dwo = moe_hip.expert_ffn_backward(
          sv["ein_y"].reshape(y_e * x_e, h0 * d_, m_), sv["h"],
          dyy.reshape(y_e * x_e, h0 * d_, n_),
          wi_s.reshape(y_e * x_e, m_, hdim), wo_s.reshape(y_e * x_e, hdim, n_),
          "relu")
      dlogits_y = moe_hip.gating_backward(
          sv["logits_y"], ry, dgate_y, dl, 1.0, router="top_2",
          importance=sv["slot_gate"].reshape(x_e * h0, t_),
          num_microbatches=gating.num_microbatches,
          importance_from_slot_gate=True,
          use_second_place_loss=gating.use_second_place_loss)
      inputs_y = sv["inputs_y"]                           # [x, h0*t, m]
      dl_y = dlogits_y.reshape(x_e, h0 * t_, y_e)
      dw_inner = torch.stack([
          moe_hip.router_backward_weights(inputs_y[i], dl_y[i])
          for i in range(x_e)])                           # [x, m, y]
      d_inputs_y = moe_hip.dispatch_backward(
          dein_y.reshape(y_e, x_e * h0, d_, m_), ry, t_, dlogits_y,
          sv["w_inner_packed"], w_gate=sv["w_inner"])
      dlogits_x = moe_hip.gating_backward(
          sv["logits_x"], rx, dgate_x, dl, 1.0, router="top_2",
          importance=sv["importance"],
          num_microbatches=gating.num_microbatches,
          use_second_place_loss=gating.use_second_place_loss)
      dw_outer = moe_hip.router_backward_weights(
          sv["x"].reshape(ag * s_, m_), dlogits_x.reshape(ag * s_, x_e))
      dx = moe_hip.dispatch_backward(
          d_inputs_y.reshape(x_e, ag, c_, m_), rx, s_, dlogits_x,
          sv["w_outer_packed"], w_gate=sv["w_outer"])
      return (dx.reshape(a0, g1, s_, m_), dw_outer, dw_inner,
              dwi.reshape(wi_s.shape), dwo.reshape(wo_s.shape))

    ins = self.inputs
    outs = mesh_impl.slicewise(fn, lowering.tensors[ins[3]],
                               lowering.tensors[ins[4]],
                               lowering.tensors[ins[5]],
                               lowering.tensors[ins[6]])
    _release_saved(lowering.operations[fwd])
    for t, v in zip(self.outputs, outs):
      lowering.set_tensor_lowering(t, v)


def transformer_moe_layer_v2(
    inputs, output_dim, hparams, train, variable_dtype,
    layout=None, mesh_shape=None, nonpadding=None, num_microbatches=None):
  """2-level mixture of experts: hparams.moe_num_experts = [x, y]; a position
  goes to up to two expert groups and, inside each, to up to two experts
  (one for its second-choice group).

  Args:
    inputs: a mtf.Tensor with shape [a, b, l, m] (or [b, l, m])
    output_dim: a mtf.Dimension (for Transformer, this is input_dim)
    hparams: model hyperparameters (those of transformer_moe_layer_v1 plus
      moe_capacity_factor_second_level)
    train: a boolean
    variable_dtype: a mtf.VariableDType
    layout: optional - an input to mtf.convert_to_layout_rules
    mesh_shape: optional - an input to mtf.convert_to_shape
    nonpadding: an optional mtf.Tensor with shape [a, b, l]
      and the same dtype as inputs, consisting of ones(nonpadding)
      and zeros(padding).
    num_microbatches: number of microbatches.

  Returns:
    outputs: a Tensor with shape [a, b, l, n]
    loss: a mtf scalar

  Raises:
    ValueError: on unrecognized hparams.moe_gating
  """
  if nonpadding is not None:
    nonpadding = mtf.zeros(inputs.mesh, inputs.shape.dims[:-1],
                           dtype=inputs.dtype) + nonpadding
  insert_outer_batch_dim = (len(inputs.shape.dims) == 3)
  if insert_outer_batch_dim:
    inputs = mtf.reshape(
        inputs, [mtf.Dimension("outer_batch", 1)] + inputs.shape.dims)

  assert len(hparams.moe_num_experts) == 2
  a0, b1, l, m = inputs.shape.dims
  hidden_dim = mtf.Dimension("expert_hidden", hparams.moe_hidden_size)
  x1 = mtf.Dimension("expert_x", hparams.moe_num_experts[0])
  y0 = mtf.Dimension("expert_y", hparams.moe_num_experts[1])
  x = mtf.Dimension("expert_x_unsplit", hparams.moe_num_experts[0])
  y = mtf.Dimension("expert_y_unsplit", hparams.moe_num_experts[1])
  n = output_dim

  num_groups, group_size = _split_into_groups(
      b1.size * l.size, hparams.moe_group_size,
      mtf.tensor_dim_to_mesh_dim_size(layout, mesh_shape, b1))
  g1 = mtf.Dimension(b1.name, num_groups)
  s = mtf.Dimension("group_size_x", group_size)
  capacity_factor = (hparams.moe_capacity_factor_train if train
                     else hparams.moe_capacity_factor_eval)
  c = mtf.Dimension("expert_capacity_x", _expert_capacity(
      s.size, capacity_factor, x.size, hparams.moe_min_expert_capacity))

  num_groups, group_size = _split_into_groups(
      a0.size * g1.size * c.size, hparams.moe_group_size,
      mtf.tensor_dim_to_mesh_dim_size(layout, mesh_shape, a0))
  t = mtf.Dimension("group_size_y", group_size)
  h0 = mtf.Dimension(a0.name, num_groups)
  d = mtf.Dimension("expert_capacity_y", _expert_capacity(
      t.size, hparams.moe_capacity_factor_second_level, y.size,
      hparams.moe_min_expert_capacity))

  inputs = mtf.reshape(inputs, [a0, g1, s, m])
  if nonpadding is not None:
    nonpadding = mtf.reshape(nonpadding, [a0, g1, s])

  if hparams.moe_gating != "top_2":
    raise ValueError("unknown hparams.moe_gating=%s" % hparams.moe_gating)
  gating = _GatingSpec(hparams, train, num_microbatches)

  w_outer = mtf_layers.get_dense_kernel_weights(
      inputs, [x], [m], [], None, name="outer_gating",
      variable_dtype=variable_dtype)
  w_inner = mtf_layers.get_dense_kernel_weights(
      inputs, [y], [m], [x1], None, name="inner_gating",
      variable_dtype=variable_dtype)
  wi = mtf_layers.get_dense_kernel_weights(
      inputs, [hidden_dim], [m], [y0, x1], None, name="wi",
      variable_dtype=variable_dtype)
  wo = mtf_layers.get_dense_kernel_weights(
      inputs, [n], [hidden_dim], [y0, x1], None, name="wo",
      variable_dtype=variable_dtype)

  output, loss = MoEV2Operation(
      inputs, w_outer, w_inner, wi, wo, nonpadding, n,
      (x.size, y.size, c.size, h0.size, t.size, d.size), gating).outputs
  output = mtf.reshape(output, [a0, b1, l, n])
  if insert_outer_batch_dim:
    output = mtf.reshape(output, [b1, l, n])
  return output, loss * hparams.moe_loss_coef


class MoE1D(transformer.TransformerLayer):
  """Mixture of Experts Layer (transformer layer adapter, moe.py:37-128)."""

  def __init__(self,
               num_experts=16,
               loss_coef=1e-2,
               hidden_size=4096,
               group_size=1024,
               capacity_factor_train=1.25,
               capacity_factor_eval=2.0,
               use_second_place_loss=False,
               second_policy_train="random",
               second_policy_eval="random",
               second_threshold_train=0.2,
               second_threshold_eval=0.2,
               dropout_rate=0.0,
               activation="relu",
               moe_gating="top_2",
               min_expert_capacity=4,
               switch_policy_train="input_jitter",
               switch_policy_eval="input_jitter",
               switch_dropout=0.1,
               switch_temperature=1.0,
               switch_jitter=1e-2,
               ntlb_top_k=4,
               output_dim=None,
               use_experts_attention=False,
               z_loss=None):
    self._hparams = HParams(
        moe_gating=moe_gating,
        moe_num_experts=num_experts,
        moe_loss_coef=loss_coef,
        moe_hidden_size=hidden_size,
        moe_group_size=group_size,
        moe_min_expert_capacity=min_expert_capacity,
        moe_capacity_factor_train=capacity_factor_train,
        moe_capacity_factor_eval=capacity_factor_eval,
        moe_use_second_place_loss=use_second_place_loss,
        moe_second_policy_train=second_policy_train,
        moe_second_policy_eval=second_policy_eval,
        moe_second_threshold_train=second_threshold_train,
        moe_second_threshold_eval=second_threshold_eval,
        moe_dropout_rate=dropout_rate,
        moe_switch_policy_train=switch_policy_train,
        moe_switch_policy_eval=switch_policy_eval,
        moe_switch_dropout=switch_dropout,
        moe_switch_temperature=switch_temperature,
        moe_switch_jitter=switch_jitter,
        moe_output_dim=output_dim,
        moe_ntlb_top_k=ntlb_top_k,
        moe_use_experts_attention=use_experts_attention,
        moe_z_loss=z_loss)
    self._activation = activation

  def call(self, context, x, losses=None):
    """Call the layer.  `context` supplies model.ensemble_dim, length_dim,
    model.model_dim/layout/mesh_shape, train, variable_dtype, nonpadding,
    num_microbatches and the `losses` list the balancing loss is appended to."""
    del losses
    if context.model.ensemble_dim:
      raise NotImplementedError("MoE not yet implemented with ensembles")
    has_length_dim = context.length_dim in x.shape.dims
    if not has_length_dim:
      x_shape = x.shape
      shape_with_length = mtf.Shape(
          x_shape.dims[:-1] + [mtf.Dimension("length", 1)] + x_shape.dims[-1:])
      x = mtf.reshape(x, shape_with_length)
    if self._hparams.moe_output_dim is not None:
      output_dim = self._hparams.moe_output_dim
    else:
      output_dim = context.model.model_dim
    y, loss = transformer_moe_layer_v1(
        x, output_dim, self._hparams, context.train, context.variable_dtype,
        layout=context.model.layout, mesh_shape=context.model.mesh_shape,
        nonpadding=context.nonpadding, activation=self._activation,
        num_microbatches=context.num_microbatches)
    if context.losses is not None:
      context.losses.append(loss)
    if not has_length_dim:
      if self._hparams.moe_use_experts_attention:
        y = [mtf.reshape(y_out, x_shape) for y_out in y]
      else:
        y = mtf.reshape(y, x_shape)
    return y


class MoE2D(transformer.TransformerLayer):
  """Hierarchical Mixture of Experts Layer (moe.py:131-188).  Unlike the
  reference's constructor this one also sets moe_min_expert_capacity (= 4, the
  MoE1D default), which transformer_moe_layer_v2 reads."""

  def __init__(self,
               expert_x=8,
               expert_y=8,
               loss_coef=1e-2,
               hidden_size=4096,
               group_size=1024,
               capacity_factor_train=1.25,
               capacity_factor_eval=2.0,
               capacity_factor_second_level=1.0,
               use_second_place_loss=False,
               second_policy_train="random",
               second_policy_eval="random",
               second_threshold_train=0.2,
               second_threshold_eval=0.2):
    self._hparams = HParams(
        moe_gating="top_2",
        moe_num_experts=[expert_x, expert_y],
        moe_loss_coef=loss_coef,
        moe_hidden_size=hidden_size,
        moe_group_size=group_size,
        moe_min_expert_capacity=4,
        moe_capacity_factor_train=capacity_factor_train,
        moe_capacity_factor_eval=capacity_factor_eval,
        moe_capacity_factor_second_level=capacity_factor_second_level,
        moe_use_second_place_loss=use_second_place_loss,
        moe_second_policy_train=second_policy_train,
        moe_second_policy_eval=second_policy_eval,
        moe_second_threshold_train=second_threshold_train,
        moe_second_threshold_eval=second_threshold_eval)

  def call(self, context, x, losses=None):
    """Call the layer."""
    del losses
    if context.model.ensemble_dim:
      raise NotImplementedError("MoE not yet implemented with ensembles")
    has_length_dim = context.length_dim in x.shape.dims
    if not has_length_dim:
      x_shape = x.shape
      shape_with_length = mtf.Shape(
          x_shape.dims[:-1] + [mtf.Dimension("length", 1)] + x_shape.dims[-1:])
      x = mtf.reshape(x, shape_with_length)
    y, loss = transformer_moe_layer_v2(
        x, context.model.model_dim, self._hparams, context.train,
        context.variable_dtype, layout=context.model.layout,
        mesh_shape=context.model.mesh_shape, nonpadding=context.nonpadding,
        num_microbatches=context.num_microbatches)
    if context.losses is not None:
      context.losses.append(loss)
    if not has_length_dim:
      y = mtf.reshape(y, x_shape)
    return y
