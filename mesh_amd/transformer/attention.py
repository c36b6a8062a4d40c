"""Multi-head attention parameters and the attention function, as
mesh_tensorflow/transformer/attention.py defines them, for the case
SelfAttention uses by default: heads and d_kv combined in the variables
(combine_dims, attention.py:410-414), separate k and v, float32 logits.
"""

import math

import numpy as np
import torch

from mesh_amd import layers as mtf_layers
from mesh_amd import ops as mtf


class AttentionParams(object):
  """The q, k, v, o kernels of multi-head attention (attention.py:345-591).

  Variables "q", "k", "v" (with shared_kv: "q", "kv") of shape
  [d_model, heads * d_kv] and "o" of shape
  [heads * d_kv, d_model]; the combined dim carries the name of its first
  member ("heads", attention.py:695-696).  Initialisers as the reference's
  without the unit-scaling convention (attention.py:436-443): q
  N(0, (d_model * d_kv)^-1) when the 1/sqrt(d_kv) scaling is folded in, k and v
  N(0, 1/d_model), o N(0, 1/(heads * d_kv)).
  """

  def __init__(self, mesh, query_input_dim, memory_input_dim, output_dim,
               key_dim, value_dim, query_heads_dims, memory_heads_dims,
               variable_dtype, shared_kv=False, no_query=False,
               combine_dims=True, ensemble_dim=None,
               keep_query_heads_dims=False,
               fold_scaling_into_initializer=True, make_attention_vars=True):
    if no_query or not combine_dims or ensemble_dim or keep_query_heads_dims:
      raise NotImplementedError(
          "only the default attention parameters are implemented (combined "
          "dims, no ensemble)")
    if key_dim != value_dim:
      raise NotImplementedError("key_dim != value_dim")
    query_heads_dims = list(query_heads_dims or [])
    memory_heads_dims = list(memory_heads_dims or [])
    if query_heads_dims != memory_heads_dims or len(query_heads_dims) > 1:
      raise NotImplementedError("memory heads other than the query heads")
    self.mesh = mesh
    self.query_input_dim = query_input_dim
    self.memory_input_dim = memory_input_dim
    self.output_dim = output_dim
    self.key_dim = key_dim
    self.value_dim = value_dim
    self.query_heads_dims = query_heads_dims
    self.memory_heads_dims = memory_heads_dims
    self.variable_dtype = variable_dtype
    self.shared_kv = shared_kv
    self.make_attention_vars = make_attention_vars
    self.fold_scaling_into_initializer = fold_scaling_into_initializer
    self.num_heads = query_heads_dims[0].size if query_heads_dims else 1
    first = (query_heads_dims + [key_dim])[0].name
    combined = mtf.Dimension(first, self.num_heads * key_dim.size)
    self.combined_dim = combined
    stddev = query_input_dim.size ** -0.5
    if fold_scaling_into_initializer:
      stddev *= key_dim.size ** -0.5
    kv_std = memory_input_dim.size ** -0.5
    o_std = combined.size ** -0.5

    normal = mtf_layers.random_normal_initializer
    # the q / k / v kernels are not needed by ExpertsAttention
    # (attention.py:443-468)
    if make_attention_vars:
      self.wq = mtf.get_variable(mesh, "q", [query_input_dim, combined],
                                 initializer=normal(stddev),
                                 dtype=variable_dtype)
      if shared_kv:                          # attention.py:453-459
        self.wkv = mtf.get_variable(mesh, "kv", [memory_input_dim, combined],
                                    initializer=normal(kv_std),
                                    dtype=variable_dtype)
      else:
        self.wk = mtf.get_variable(mesh, "k", [memory_input_dim, combined],
                                   initializer=normal(kv_std),
                                   dtype=variable_dtype)
        self.wv = mtf.get_variable(mesh, "v", [memory_input_dim, combined],
                                   initializer=normal(kv_std),
                                   dtype=variable_dtype)
    self.wo = mtf.get_variable(mesh, "o", [combined, output_dim],
                               initializer=normal(o_std), dtype=variable_dtype)

  def _project(self, x, w, name):
    return mtf_layers.DenseOperation(x, w, [w.shape.dims[-1]], None,
                                     name=name).outputs[0]

  def compute_q(self, query_antecedent):
    """[..., d_model] -> [..., heads * d_kv] (attention.py:481-497)."""
    q = self._project(query_antecedent, self.wq, "q_proj")
    if not self.fold_scaling_into_initializer:
      q = q * (self.key_dim.size ** -0.5)
    return q

  def compute_kv(self, memory_antecedent):
    """The tensor that serves as keys and as values (attention.py:499-515)."""
    if not self.shared_kv:
      raise ValueError("compute_kv can only be called with shared_kv")
    return self._project(memory_antecedent, self.wkv, "kv_proj")

  def compute_k(self, memory_antecedent):
    if self.shared_kv:
      raise ValueError("compute_k cannot be called with shared_kv")
    return self._project(memory_antecedent, self.wk, "k_proj")

  def compute_v(self, memory_antecedent):
    if self.shared_kv:
      raise ValueError("compute_v cannot be called with shared_kv")
    return self._project(memory_antecedent, self.wv, "v_proj")

  def compute_output(self, o, output_shape=None):
    """[..., heads * d_kv] -> [..., d_model] (attention.py:553-575)."""
    y = self._project(o, self.wo, "o_proj")
    if output_shape is not None and y.shape != mtf.convert_to_shape(
        output_shape):
      raise ValueError("attention output %s, expected %s"
                       % (y.shape, output_shape))
    return y


class ExpertsAttentionParams(AttentionParams):
  """Attention parameters whose queries and keys come out of a
  Mixture-of-Experts layer (attention.py:594-692): a MoE1D with
  use_experts_attention projects the antecedent to [q, k] through two output
  kernels of the same experts ("q_wo", "k_wo"), the keys are also the values
  (shared_kv) and only the output kernel "o" is a variable of its own.  The
  queries are scaled by d_kv ** -0.5 after the layer (attention.py:664-665).

  The reference passes `switch_top_k` to a MoE1D constructor that has no such
  argument (transformer/moe.py:44-66), so its version cannot be constructed;
  here the value goes to `ntlb_top_k`, the only top-k the layer has."""

  def __init__(self, mesh, query_input_dim, memory_input_dim, output_dim,
               key_dim, value_dim, query_heads_dims, memory_heads_dims,
               variable_dtype, shared_kv=False, no_query=False,
               combine_dims=True, ensemble_dim=None,
               keep_query_heads_dims=False,
               fold_scaling_into_initializer=True, context=None,
               experts_hparams=None):
    super(ExpertsAttentionParams, self).__init__(
        mesh=mesh, query_input_dim=query_input_dim,
        memory_input_dim=memory_input_dim, output_dim=output_dim,
        key_dim=key_dim, value_dim=value_dim,
        query_heads_dims=query_heads_dims, memory_heads_dims=memory_heads_dims,
        variable_dtype=variable_dtype, shared_kv=shared_kv, no_query=no_query,
        combine_dims=combine_dims, ensemble_dim=ensemble_dim,
        keep_query_heads_dims=keep_query_heads_dims,
        fold_scaling_into_initializer=fold_scaling_into_initializer,
        make_attention_vars=False)
    self.context = context
    if not combine_dims:
      raise ValueError("self.combine_dims must be True for ExpertsAttention")
    if not shared_kv:
      raise ValueError("self.shared_kv must be True for ExpertsAttention")
    from mesh_amd.transformer import moe
    hp = experts_hparams
    self.moe_layer = moe.MoE1D(
        moe_gating=hp.moe_gating, num_experts=hp.num_experts,
        loss_coef=hp.loss_coef, group_size=hp.group_size,
        min_expert_capacity=hp.min_expert_capacity,
        capacity_factor_train=hp.capacity_factor_train,
        capacity_factor_eval=hp.capacity_factor_eval,
        switch_policy_train=hp.switch_policy_train,
        switch_policy_eval=hp.switch_policy_eval,
        switch_dropout=hp.switch_dropout,
        switch_temperature=hp.switch_temperature,
        switch_jitter=hp.switch_jitter, ntlb_top_k=hp.switch_top_k,
        hidden_size=hp.hidden_size, output_dim=self.combined_dim,
        use_experts_attention=hp.use_experts_attention)
    self._q = self._k = None

  def _compute_merge_qkv(self, antecedent):
    """q and k in one call of the experts layer (query and memory antecedent
    are taken to be the same, attention.py:657-667)."""
    q, k = self.moe_layer.call(self.context, antecedent)
    self._q = q * (self.key_dim.size ** -0.5)
    self._k = k

  def compute_q(self, query_antecedent):
    self._compute_merge_qkv(query_antecedent)
    return self._q

  def compute_k(self, memory_antecedent):
    del memory_antecedent
    return self._k

  def compute_kv(self, memory_antecedent):
    del memory_antecedent
    return self._k

  def compute_v(self, memory_antecedent):
    del memory_antecedent
    raise NotImplementedError("ExpertsAttention uses shared_kv = True.")


def relative_position_bucket(relative_position, bidirectional=True,
                             num_buckets=32, max_distance=128):
  """_relative_position_bucket (transformer_layers.py:1000-1042) on host
  integers: relative_position = memory position - query position -> bucket in
  [0, num_buckets).  Half of the buckets hold exact small distances, the rest
  grow logarithmically up to max_distance; the logarithmic part is float32
  arithmetic in the reference's op order, truncated as its int32 cast does."""
  rp = np.asarray(relative_position, np.int64)
  ret = np.zeros(rp.shape, np.int64)
  n = -rp
  if bidirectional:
    num_buckets //= 2
    ret = ret + (n < 0) * num_buckets
    n = np.abs(n)
  else:
    n = np.maximum(n, 0)
  max_exact = num_buckets // 2
  is_small = n < max_exact
  safe = np.where(is_small, max_exact, n).astype(np.float32)
  scaled = (np.log(safe / np.float32(max_exact)).astype(np.float32)
            / np.float32(math.log(max_distance / max_exact))
            ).astype(np.float32) * np.float32(num_buckets - max_exact)
  large = np.minimum(max_exact + scaled.astype(np.int64), num_buckets - 1)
  return ret + np.where(is_small, n, large)


class SelfAttentionOperation(mtf.Operation):
  """attention.attention (attention.py:27-88) on combined-dim tensors
  q, k, v [batch..., length, heads * d_kv]: float32 logits, an optional
  autoregressive visibility mask, float32 softmax, weights in the activation
  dtype, weights . v.  sequence_id [batch..., length] (int32) restricts a
  query to the keys of its own sequence (the bias of
  transformer_layers.py:303-316)."""

  def __init__(self, q, k, v, num_heads, causal, sequence_id=None,
               relative_values=None, relative_bidirectional=True, name=None):
    inputs = [q, k, v] + ([] if sequence_id is None else [sequence_id]) + (
        [] if relative_values is None else [relative_values])
    super(SelfAttentionOperation, self).__init__(inputs,
                                                 name=name or "attention")
    self._ids_at = 3 if sequence_id is not None else None
    self._rel_at = (len(inputs) - 1) if relative_values is not None else None
    self._rel_bidirectional = bool(relative_bidirectional)
    if relative_values is not None and (
        relative_values.shape.ndims != 2
        or relative_values.shape.dims[0].size != num_heads):
      raise ValueError("relative attention bias %s, expected [heads = %d, "
                       "buckets]" % (relative_values.shape, num_heads))
    if q.shape != k.shape or q.shape != v.shape:
      raise ValueError("q, k, v shapes differ: %s %s %s"
                       % (q.shape, k.shape, v.shape))
    if sequence_id is not None and (
        sequence_id.shape.dims != q.shape.dims[:-1]):
      raise ValueError("sequence_id %s does not match q %s"
                       % (sequence_id.shape, q.shape))
    self._num_heads = num_heads
    self._causal = bool(causal)
    self._save_for_backward = False     # set once a gradient is asked for
    self._outputs = [mtf.Tensor(self, q.shape, q.dtype)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    sizes = self.outputs[0].shape.to_integer_list
    length, channels = sizes[-2], sizes[-1]
    heads, causal = self._num_heads, self._causal

    ids_at, rel_at = self._ids_at, self._rel_at
    bidirectional = self._rel_bidirectional

    def fn(q, k, v, *extra):
      q3, k3, v3 = (t.reshape(-1, length, channels).contiguous()
                    for t in (q, k, v))
      ids, rel = _attention_extras(extra, ids_at, rel_at, length, bidirectional,
                                   q.dtype)
      # a backward pass follows: where the fused kernels run, keep the softmax
      # denominators (and the outputs) so that it need not recompute them
      if self._save_for_backward and moe_hip.fused_attention_applies(q3, heads):
        out, lse = moe_hip.self_attention(q3, k3, v3, heads, causal,
                                          sequence_id=ids, relative_bias=rel,
                                          return_lse=True)
        saved.update(out=out, lse=lse)
        return out.reshape(sizes)
      return moe_hip.self_attention(q3, k3, v3, heads, causal, sequence_id=ids,
                                    relative_bias=rel).reshape(sizes)
    saved = {}
    lowering.set_tensor_lowering(
        self.outputs[0],
        mesh_impl.slicewise(fn, *[lowering.tensors[t] for t in self.inputs]))
    lowering.operations[self] = saved

  def gradient(self, grad_ys):
    self._save_for_backward = True
    grads = list(SelfAttentionGradOperation(self, grad_ys[0]).outputs)
    out = grads[:3] + [None] * (len(self.inputs) - 3)
    if self._rel_at is not None:
      out[self._rel_at] = grads[3]
    return out


# The bucket of every (memory position - query position) of a length, as a
# device tensor: built once per (length, direction, bucket count, device) and
# kept, so that a lowering -- in particular every decoding step, and a step
# being recorded into a HIP graph, where a host-to-device copy from pageable
# memory cannot be captured -- only indexes it.
_BUCKET_TABLES = {}


def relative_bucket_table(length, bidirectional, num_buckets, device):
  """int32 [2 * length - 1] on `device`: entry d is the bucket of the distance
  d - (length - 1)."""
  key = (int(length), bool(bidirectional), int(num_buckets), str(device))
  table = _BUCKET_TABLES.get(key)
  if table is None:
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
      raise RuntimeError(
          "the relative-position bucket table for length %d is not on the "
          "device yet and cannot be uploaded while a HIP graph is being "
          "recorded: run the step once before capturing it" % length)
    bucket = relative_position_bucket(
        np.arange(-(length - 1), length), bidirectional, num_buckets)
    table = torch.from_numpy(bucket.astype(np.int32)).to(device)
    _BUCKET_TABLES[key] = table
  return table


def _attention_extras(extra, ids_at, rel_at, length, bidirectional, dtype):
  """The optional inputs of the attention operations as the library takes
  them: sequence ids [B, L] int32, and (bias values [H, NB] in the activation
  dtype, the bucket of every memory position - query position [2L-1])."""
  ids = rel = None
  if ids_at is not None:
    ids = extra[ids_at - 3].reshape(-1, length).to(torch.int32).contiguous()
  if rel_at is not None:
    values = extra[rel_at - 3].to(dtype).contiguous()
    rel = (values, relative_bucket_table(length, bidirectional,
                                         values.shape[-1], values.device))
  return ids, rel


class AttentionDecodeOperation(mtf.Operation):
  """One decoding step of self-attention (SelfAttention.call in "incremental"
  mode, transformer_layers.py:231-254): q, k, v [batch..., heads * d_kv] of the
  step, the recurrent states old_k, old_v [batch..., memory_length,
  heads * d_kv] and position [batch...] (int32) -> the attention outputs
  [batch..., heads * d_kv] and the updated states.  The states are new tensors
  (the graph stays functional); the library call updates a copy in place.
  relative_values [heads, buckets]: the relative attention bias of the memory
  positions against the step's position (transformer_layers.py:317-352)."""

  def __init__(self, q, k, v, old_k, old_v, position, num_heads,
               relative_values=None, relative_bidirectional=False, name=None):
    super(AttentionDecodeOperation, self).__init__(
        [q, k, v, old_k, old_v, position] + (
            [] if relative_values is None else [relative_values]),
        name=name or "attention_decode")
    self._rel_bidirectional = bool(relative_bidirectional)
    if q.shape != k.shape or q.shape != v.shape or old_k.shape != old_v.shape:
      raise ValueError("q, k, v %s %s %s / states %s %s"
                       % (q.shape, k.shape, v.shape, old_k.shape, old_v.shape))
    if (old_k.shape.dims[:-2] != q.shape.dims[:-1]
        or old_k.shape.dims[-1] != q.shape.dims[-1]
        or position.shape.dims != q.shape.dims[:-1]):
      raise ValueError("states %s / position %s do not match q %s"
                       % (old_k.shape, position.shape, q.shape))
    self._num_heads = num_heads
    self._outputs = [mtf.Tensor(self, q.shape, q.dtype, index=0),
                     mtf.Tensor(self, old_k.shape, old_k.dtype, index=1),
                     mtf.Tensor(self, old_v.shape, old_v.dtype, index=2)]

  has_gradient = False

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    q_sizes = self.outputs[0].shape.to_integer_list
    s_sizes = self.outputs[1].shape.to_integer_list
    channels, memory = q_sizes[-1], s_sizes[-2]
    heads = self._num_heads

    bidirectional = self._rel_bidirectional

    def fn(q, k, v, old_k, old_v, position, *extra):
      q2, k2, v2 = (t.reshape(-1, channels).contiguous() for t in (q, k, v))
      kc = old_k.reshape(-1, memory, channels).clone()
      vc = old_v.reshape(-1, memory, channels).clone()
      pos = position.reshape(-1).to(torch.int32).contiguous()
      _, rel = _attention_extras(extra, None, 3 if extra else None, memory,
                                 bidirectional, q.dtype)
      out = moe_hip.attention_decode(q2, k2, v2, kc, vc, pos, heads,
                                     relative_bias=rel)
      return out.reshape(q_sizes), kc.reshape(s_sizes), vc.reshape(s_sizes)
    outs = mesh_impl.slicewise(fn, *[lowering.tensors[t] for t in self.inputs])
    for tensor, value in zip(self.outputs, outs):
      lowering.set_tensor_lowering(tensor, value)


class SelfAttentionGradOperation(mtf.Operation):
  """(dq, dk, dv) of a SelfAttentionOperation: the gradients of the two
  einsums and the softmax of attention.attention (attention.py:76-87), with
  the weights recomputed."""

  def __init__(self, forward, dout, name=None):
    q, k, v = forward.inputs[:3]
    super(SelfAttentionGradOperation, self).__init__(
        [dout, q, k, v] + list(forward.inputs[3:]),
        name=name or "attention_grad")
    # pylint: disable=protected-access
    self._forward = forward
    self._num_heads, self._causal = forward._num_heads, forward._causal
    self._ids_at, self._rel_at = forward._ids_at, forward._rel_at
    self._rel_bidirectional = forward._rel_bidirectional
    wrt = [q, k, v] + ([] if self._rel_at is None
                       else [forward.inputs[self._rel_at]])
    self._outputs = [mtf.Tensor(self, t.shape, t.dtype, index=i)
                     for i, t in enumerate(wrt)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    sizes = self.outputs[0].shape.to_integer_list
    length, channels = sizes[-2], sizes[-1]
    heads, causal = self._num_heads, self._causal

    ids_at, rel_at = self._ids_at, self._rel_at
    bidirectional = self._rel_bidirectional

    def fn(dout, q, k, v, *extra):
      d3, q3, k3, v3 = (t.reshape(-1, length, channels).contiguous()
                        for t in (dout, q, k, v))
      ids, rel = _attention_extras(extra, ids_at, rel_at, length, bidirectional,
                                   q.dtype)
      saved = lowering.operations.get(self._forward) or {}
      grads = moe_hip.self_attention_backward(
          q3, k3, v3, d3, heads, causal, sequence_id=ids, relative_bias=rel,
          out=saved.get("out"), lse=saved.get("lse"))
      saved.clear()
      return tuple(t.reshape(sizes) for t in grads[:3]) + tuple(grads[3:])
    grads = mesh_impl.slicewise(
        fn, *[lowering.tensors[t] for t in self.inputs])
    for out, value in zip(self.outputs, grads):
      lowering.set_tensor_lowering(out, value)
