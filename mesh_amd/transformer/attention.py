"""Multi-head attention parameters and the attention function, as
mesh_tensorflow/transformer/attention.py defines them, for the case
SelfAttention uses by default: heads and d_kv combined in the variables
(combine_dims, attention.py:410-414), separate k and v, float32 logits.
"""

from mesh_amd import layers as mtf_layers
from mesh_amd import ops as mtf


class AttentionParams(object):
  """The q, k, v, o kernels of multi-head attention (attention.py:345-591).

  Variables "q", "k", "v" of shape [d_model, heads * d_kv] and "o" of shape
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
    if shared_kv or no_query or not combine_dims or ensemble_dim or \
        keep_query_heads_dims or not make_attention_vars:
      raise NotImplementedError(
          "only the default attention parameters are implemented (separate "
          "k and v, combined dims, no ensemble)")
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
    self.wq = mtf.get_variable(mesh, "q", [query_input_dim, combined],
                               initializer=normal(stddev), dtype=variable_dtype)
    self.wk = mtf.get_variable(mesh, "k", [memory_input_dim, combined],
                               initializer=normal(kv_std), dtype=variable_dtype)
    self.wv = mtf.get_variable(mesh, "v", [memory_input_dim, combined],
                               initializer=normal(kv_std), dtype=variable_dtype)
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

  def compute_k(self, memory_antecedent):
    return self._project(memory_antecedent, self.wk, "k_proj")

  def compute_v(self, memory_antecedent):
    return self._project(memory_antecedent, self.wv, "v_proj")

  def compute_output(self, o, output_shape=None):
    """[..., heads * d_kv] -> [..., d_model] (attention.py:553-575)."""
    y = self._project(o, self.wo, "o_proj")
    if output_shape is not None and y.shape != mtf.convert_to_shape(
        output_shape):
      raise ValueError("attention output %s, expected %s"
                       % (y.shape, output_shape))
    return y


class SelfAttentionOperation(mtf.Operation):
  """attention.attention (attention.py:27-88) on combined-dim tensors
  q, k, v [batch..., length, heads * d_kv]: float32 logits, an optional
  autoregressive visibility mask, float32 softmax, weights in the activation
  dtype, weights . v."""

  def __init__(self, q, k, v, num_heads, causal, name=None):
    super(SelfAttentionOperation, self).__init__([q, k, v],
                                                 name=name or "attention")
    if q.shape != k.shape or q.shape != v.shape:
      raise ValueError("q, k, v shapes differ: %s %s %s"
                       % (q.shape, k.shape, v.shape))
    self._num_heads = num_heads
    self._causal = bool(causal)
    self._outputs = [mtf.Tensor(self, q.shape, q.dtype)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    sizes = self.outputs[0].shape.to_integer_list
    length, channels = sizes[-2], sizes[-1]
    heads, causal = self._num_heads, self._causal

    def fn(q, k, v):
      q3, k3, v3 = (t.reshape(-1, length, channels).contiguous()
                    for t in (q, k, v))
      return moe_hip.self_attention(q3, k3, v3, heads, causal).reshape(sizes)
    lowering.set_tensor_lowering(
        self.outputs[0],
        mesh_impl.slicewise(fn, *[lowering.tensors[t] for t in self.inputs]))
