"""DenseReluDense and SelfAttention as mesh_tensorflow/transformer/
transformer_layers.py defines them, for training / evaluation on one device.
"""

from mesh_amd import layers as mtf_layers
from mesh_amd import ops as mtf
from mesh_amd.transformer import attention
from mesh_amd.transformer import transformer


class DenseReluDense(transformer.TransformerLayer):
  """Two dense layers with an activation on the hidden layer
  (transformer_layers.py:36-76): variables wi/kernel [d_model, d_ff] and
  wo/kernel [d_ff, d_model]."""

  def __init__(self, hidden_size=4096, dropout_rate=0.0, activation="relu",
               use_bias=False):
    self.hidden_size = hidden_size
    self.dropout_rate = dropout_rate
    self.activation = activation
    self.use_bias = use_bias

  def call(self, context, x, losses=None):
    del losses
    io_channels = x.shape.dims[-1]
    hidden_channels = mtf.Dimension("d_ff", self.hidden_size)
    if context.model.ensemble_dims:
      raise NotImplementedError("ensembles are not implemented")
    h = mtf_layers.dense_product(
        x, reduced_dims=x.shape.dims[-1:], new_dims=hidden_channels,
        activation_functions=self.activation, use_bias=self.use_bias,
        variable_dtype=context.variable_dtype, name="wi")
    if context.train and self.dropout_rate != 0.0:   # transformer_layers.py:67-69
      h = mtf.dropout(h, context.train, keep_prob=1.0 - self.dropout_rate,
                      noise_shape=h.shape - context.length_dim)
    y = mtf_layers.dense(
        h, io_channels, use_bias=self.use_bias, activation=None,
        variable_dtype=context.variable_dtype, reduced_dims=h.shape.dims[-1:],
        name="wo")
    return y


class SelfAttention(transformer.TransformerLayer):
  """Multi-head self-attention (transformer_layers.py:151-357): combined dims,
  separate k and v kernels or one for both (shared_kv), optionally the relative
  position bias of types "bias" and "bias_shared".  Visibility comes from the
  context: read/write priorities (autoregressive models), sequence ids, or
  none."""

  def __init__(self, num_heads=8, num_memory_heads=0, key_value_size=128,
               shared_kv=False, dropout_rate=0.0, attention_kwargs=None,
               relative_attention_type=None,
               relative_attention_num_buckets=32, attention_func=None,
               combine_dims=True, keep_query_heads_dims=False,
               fold_scaling_into_initializer=True):
    if (num_memory_heads or attention_kwargs or attention_func is not None or
        not combine_dims or keep_query_heads_dims):
      raise NotImplementedError(
          "only the default SelfAttention options are implemented")
    if relative_attention_type == "contextual":
      raise NotImplementedError("contextual relative attention")
    if relative_attention_type not in (None, "bias", "bias_shared"):
      raise ValueError("unrecognized relative_attention_type \"%s\""
                       % relative_attention_type)
    self.relative_attention_type = relative_attention_type
    self.num_heads = num_heads
    self.shared_kv = shared_kv
    self.combine_dims = combine_dims
    self.key_value_size = key_value_size
    self.dropout_rate = dropout_rate
    self.relative_attention_num_buckets = relative_attention_num_buckets
    self.fold_scaling_into_initializer = fold_scaling_into_initializer

  @property
  def kv_dim(self):
    return mtf.Dimension("d_kv", self.key_value_size)

  def make_params(self, context):
    """transformer_layers.py:79-149 (attention_params)."""
    heads = ([mtf.Dimension("heads", self.num_heads)]
             if self.num_heads > 1 else None)
    return attention.AttentionParams(
        context.mesh, query_input_dim=context.model.model_dim,
        memory_input_dim=context.model.model_dim,
        output_dim=context.model.model_dim, key_dim=self.kv_dim,
        value_dim=self.kv_dim, query_heads_dims=heads,
        memory_heads_dims=heads, variable_dtype=context.variable_dtype,
        shared_kv=self.shared_kv, ensemble_dim=context.model.ensemble_dim,
        fold_scaling_into_initializer=self.fold_scaling_into_initializer)

  def relative_bias_values(self, context, num_heads):
    """The learned bias per (head, bucket of memory position - query position)
    (compute_bias, transformer_layers.py:317-352): the variable
    "relative_attention_bias" [heads, buckets]; with "bias_shared" the first
    layer's variable serves every layer of the stack (context.cache)."""
    if self.relative_attention_type is None:
      return None
    heads = mtf.Dimension("heads", num_heads)
    buckets = mtf.Dimension("buckets", self.relative_attention_num_buckets)
    shared = self.relative_attention_type == "bias_shared"
    key = ("self_attention_bias", None, None, (heads,))
    if shared and key in context.cache:
      return context.cache[key]
    values = mtf.get_variable(context.mesh, "relative_attention_bias",
                              mtf.Shape([heads, buckets]),
                              dtype=context.variable_dtype)
    if shared:
      context.cache[key] = values
    return values

  def _attention_dropout(self, context, v, num_heads):
    """Dropout of the attention weights with one noise value per (batch entry,
    head, memory position), shared by the queries (attention.py:82-84 with
    dropout_broadcast_dims = [length], transformer_layers.py:210-212):
    sum_k weights[b,h,q,k] * noise[b,h,k] * v[b,k,h,:] is the undropped
    attention over v * noise, so the noise goes onto the values."""
    batch_length = v.shape.dims[:-1]
    heads = mtf.Dimension("heads", num_heads)
    per_head = mtf.Dimension("d_kv", v.shape.dims[-1].size // num_heads)
    split = mtf.reshape(v, mtf.Shape(batch_length + [heads, per_head]))
    split = mtf.dropout(split, context.train, keep_prob=1.0 - self.dropout_rate,
                        noise_shape=mtf.Shape(batch_length + [heads]))
    return mtf.reshape(split, v.shape)

  def call(self, context, x, losses=None):
    """transformer_layers.py:223-271 for the train / eval modes."""
    del losses
    if isinstance(context.subsequence_id, mtf.Tensor):
      raise NotImplementedError("subsequence_id tensors are not implemented")
    # a query sees only its own sequence (transformer_layers.py:303-316)
    sequence_id = (context.sequence_id
                   if isinstance(context.sequence_id, mtf.Tensor) else None)
    params = self.make_params(context)
    q = params.compute_q(x)
    if self.shared_kv:                       # transformer_layers.py:246-249
      k = v = params.compute_kv(x)
    else:
      k = params.compute_k(x)
      v = params.compute_v(x)
    relative_values = self.relative_bias_values(context, params.num_heads)
    if context.mode == transformer.INCREMENTAL:
      # one position per batch entry: the step's key and value replace row
      # `position` of the recurrent states, the query sees the memory
      # positions up to it (transformer_layers.py:239-254, :289-296)
      if sequence_id is not None:
        raise NotImplementedError("incremental mode with sequence ids")
      if context.read_priority is not transformer.POSITION:
        raise NotImplementedError("incremental mode of a model that is not "
                                  "autoregressive")
      if self.shared_kv:                     # one state: the shared tensor
        old_k = old_v = context.get_states(1)[0]
      else:
        old_k, old_v = context.get_states(2)
      op = attention.AttentionDecodeOperation(
          q, k, v, old_k, old_v, context.position, params.num_heads,
          relative_values=relative_values,
          relative_bidirectional=not context.model.fully_autoregressive)
      o, k_all, v_all = op.outputs
      context.record_new_states([k_all] if self.shared_kv else [k_all, v_all])
      return params.compute_output(o, output_shape=x.shape)
    if context.mode == transformer.FIRST_PART:
      name = context.length_dim.name       # states carry "memory_length"
      context.record_new_states(
          [mtf.rename_dimension(t, name, "memory_length")
           for t in ([k] if self.shared_kv else [k, v])])
    # read_priority >= write_priority (transformer_layers.py:289-296)
    causal = context.read_priority is transformer.POSITION
    if context.train and self.dropout_rate != 0.0:
      v = self._attention_dropout(context, v, params.num_heads)
    o = attention.SelfAttentionOperation(
        q, k, v, params.num_heads, causal, sequence_id=sequence_id,
        relative_values=relative_values,
        # buckets of a bidirectional layout unless the model is autoregressive
        # (transformer_layers.py:321)
        relative_bidirectional=not context.model.fully_autoregressive
        ).outputs[0]
    return params.compute_output(o, output_shape=x.shape)


class ExpertsSelfAttention(SelfAttention):
  """Self-attention whose queries and keys (= values) are computed by a
  Mixture-of-Experts layer (transformer_layers.py:383-459).  `shared_kv=True`
  must be passed, as to the reference's.  Variables under the layer's scope:
  the experts layer's "<router>_gating/kernel", "wi/kernel", "q_wo/kernel",
  "k_wo/kernel" and the attention output kernel "o"."""

  def __init__(self, num_experts=16, loss_coef=1e-2, group_size=1024,
               capacity_factor_train=1.25, capacity_factor_eval=2.0,
               moe_gating="switch", min_expert_capacity=4,
               switch_policy_train="input_jitter",
               switch_policy_eval="input_jitter", switch_dropout=0.0,
               switch_temperature=1.0, switch_jitter=1e-2, switch_top_k=4,
               hidden_size=3072, use_experts_attention=True, **kwargs):
    super(ExpertsSelfAttention, self).__init__(**kwargs)
    from mesh_amd.transformer import moe
    self._hparams = moe.HParams(
        moe_gating=moe_gating, num_experts=num_experts, loss_coef=loss_coef,
        group_size=group_size, min_expert_capacity=min_expert_capacity,
        capacity_factor_train=capacity_factor_train,
        capacity_factor_eval=capacity_factor_eval,
        switch_policy_train=switch_policy_train,
        switch_policy_eval=switch_policy_eval, switch_dropout=switch_dropout,
        switch_temperature=switch_temperature, switch_jitter=switch_jitter,
        switch_top_k=switch_top_k, hidden_size=hidden_size,
        use_experts_attention=use_experts_attention)

  def make_params(self, context):
    heads = ([mtf.Dimension("heads", self.num_heads)]
             if self.num_heads > 1 else None)
    return attention.ExpertsAttentionParams(
        context.mesh, query_input_dim=context.model.model_dim,
        memory_input_dim=context.model.model_dim,
        output_dim=context.model.model_dim, key_dim=self.kv_dim,
        value_dim=self.kv_dim, query_heads_dims=heads,
        memory_heads_dims=heads, variable_dtype=context.variable_dtype,
        shared_kv=self.shared_kv, no_query=False,
        ensemble_dim=context.model.ensemble_dim,
        combine_dims=self.combine_dims,
        fold_scaling_into_initializer=self.fold_scaling_into_initializer,
        context=context, experts_hparams=self._hparams)
