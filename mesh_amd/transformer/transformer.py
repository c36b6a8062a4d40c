"""The layer-stack part of mesh_tensorflow/transformer/transformer.py that a
Mixture-of-Experts transformer block needs: TransformerLayer, Context,
LayerStack with its sublayers (RMS norm, layer call, dropout, residual,
padding mask), make_layer_stack, and the layer-stack call of Unitransformer.

Decoding: the "first_part" and "incremental" modes of the Context and of
SelfAttention (recurrent key / value states); the sampling loop around them
stays with the caller.

Not here: embeddings, vocabularies, logits and losses of Unitransformer /
Bitransformer, ensembles, subsequence ids.
"""

from mesh_amd import layers as mtf_layers
from mesh_amd import ops as mtf

TRAIN = "train"   # tf.estimator.ModeKeys.TRAIN
EVAL = "eval"     # tf.estimator.ModeKeys.EVAL
FIRST_PART = "first_part"     # decoding: the known first part, records states
INCREMENTAL = "incremental"   # decoding: one position per call, states in/out


class _Position(object):
  """Stands for mtf.range(mesh, length_dim, int32), the value Unitransformer
  gives read_priority and write_priority of an autoregressive model
  (transformer.py:1032-1040): position a sees position b iff a >= b."""

  def __repr__(self):
    return "POSITION"


POSITION = _Position()


class TransformerLayer(object):
  """Base class of the layers (transformer.py:56-105): the constructor records
  hyperparameters, call(context, x) builds the layer and its variables."""

  def call(self, context, x):
    raise NotImplementedError("Not implemented")

  def set_name(self, name):
    self._name = name

  @property
  def name(self):
    return getattr(self, "_name", None)


# Context fields that only decoding, beam search, encoder-decoder attention or
# parameter sharing use; accepted for signature compatibility, must stay None.
_UNUSED_CONTEXT_FIELDS = (
    "beam_dim", "subsequence_id", "initial_position",
    "encoder_output", "encoder_sequence_id", "constant_states",
    "shared_params", "encoder_layer_outputs", "inputs", "encoder_inputs")


class Context(object):
  """What layers need at call time (transformer.py:107-311), for the "train"
  and "eval" modes.  read_priority / write_priority are None (every position
  sees every position) or POSITION (autoregressive); sequence_id is None, 1
  (no padding) or an int32 Tensor [batch..., length] (packed sequences; 0 marks
  padding).  The reference's remaining constructor arguments
  (_UNUSED_CONTEXT_FIELDS) are accepted as keywords and must be None."""

  def __init__(self, model, mesh, batch_dims, length_dim, variable_dtype,
               mode=TRAIN, position=None, position_is_default=False,
               sequence_id=None, losses=None, layer_outputs=None,
               write_priority=None, read_priority=None, num_microbatches=1,
               states=None, new_states=None, **unused):
    if mode not in (TRAIN, EVAL, FIRST_PART, INCREMENTAL):
      raise ValueError("unknown mode %r" % (mode,))
    if mode == INCREMENTAL and not isinstance(position, mtf.Tensor):
      raise ValueError("incremental mode needs the position tensor "
                       "[batch dims] (int32)")
    for key, value in unused.items():
      if key not in _UNUSED_CONTEXT_FIELDS:
        raise TypeError("Context got an unexpected argument %r" % key)
      if value is not None:
        raise NotImplementedError("Context.%s is not implemented" % key)
    if (write_priority is None) != (read_priority is None):
      raise ValueError("read_priority and write_priority go together")
    if write_priority not in (None, POSITION) or read_priority not in (
        None, POSITION):
      raise NotImplementedError("read/write priorities other than the position")
    for key in _UNUSED_CONTEXT_FIELDS:
      setattr(self, key, None)
    self.shared_params = {}
    self.model, self.mesh = model, mesh
    self.batch_dims, self.length_dim = batch_dims, length_dim
    self.variable_dtype = variable_dtype
    self.mode = mode
    self.position, self.position_is_default = position, position_is_default
    self.sequence_id = sequence_id
    self.losses = losses
    self.layer_outputs = [] if layer_outputs is None else layer_outputs
    self.write_priority, self.read_priority = write_priority, read_priority
    self.num_microbatches = num_microbatches
    # recurrent states of decoding (transformer.py:251-272): layers read
    # theirs with get_states in "incremental" mode and append the new values
    # with record_new_states in "first_part" and "incremental" modes
    self.states = [] if states is None else list(states)
    self.new_states = [] if new_states is None else new_states
    self.layer_index = 0
    self.cache = {}            # values shared between layers

  train = property(lambda self: self.mode == TRAIN)

  def get_states(self, n):
    """The next n recurrent states (transformer.py:251-261)."""
    got = self.states[len(self.new_states):len(self.new_states) + n]
    if len(got) != n:
      raise ValueError("incremental mode: %d states were passed, a layer asks "
                       "for states %d..%d" % (len(self.states),
                                              len(self.new_states),
                                              len(self.new_states) + n - 1))
    return got

  def record_new_states(self, new_states):
    """transformer.py:263-271."""
    self.new_states.extend(new_states)
  activation_dtype = property(
      lambda self: self.variable_dtype.activation_dtype)

  @property
  def nonpadding(self):
    """Zeros in padding positions and ones elsewhere (transformer.py:297-306):
    None without a sequence_id, the integer 1 when sequence_id == 1, else
    cast(sequence_id != 0, activation dtype) (built once per context)."""
    if self.sequence_id is None:
      return None
    if isinstance(self.sequence_id, int) and self.sequence_id == 1:
      return 1
    if "nonpadding" not in self.cache:
      self.cache["nonpadding"] = mtf.cast(
          mtf.not_equal(self.sequence_id, 0), self.activation_dtype)
    return self.cache["nonpadding"]


class RmsNormOperation(mtf.Operation):
  """x * rsqrt(mean(square(x)) + epsilon) * scale over the last dim: the five
  ops of sublayer_rms_norm (transformer.py:493-516) in one kernel."""

  def __init__(self, x, scale, epsilon, name=None):
    super(RmsNormOperation, self).__init__([x, scale], name=name or "rms_norm")
    if scale.shape.dims != x.shape.dims[-1:]:
      raise ValueError("scale %s does not match the last dim of %s"
                       % (scale.shape, x.shape))
    self._epsilon = float(epsilon)
    self._outputs = [mtf.Tensor(self, x.shape, x.dtype)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    eps = self._epsilon

    def fn(x, scale):
      return moe_hip.rms_norm(x.contiguous(), scale.contiguous(), eps)
    lowering.set_tensor_lowering(
        self.outputs[0],
        mesh_impl.slicewise(fn, *[lowering.tensors[t] for t in self.inputs]))

  def gradient(self, grad_ys):
    return list(RmsNormGradOperation(self, grad_ys[0]).outputs)


class RmsNormGradOperation(mtf.Operation):
  """(dx, dscale) of an RmsNormOperation."""

  def __init__(self, forward, dy, name=None):
    x, scale = forward.inputs
    super(RmsNormGradOperation, self).__init__(
        [dy, x, scale], name=name or "rms_norm_grad")
    self._epsilon = forward._epsilon   # pylint: disable=protected-access
    self._outputs = [mtf.Tensor(self, x.shape, x.dtype, index=0),
                     mtf.Tensor(self, scale.shape, scale.dtype, index=1)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    eps = self._epsilon

    def fn(dy, x, scale):
      dx, dscale = moe_hip.rms_norm_backward(
          x.contiguous(), scale.to(x.dtype).contiguous(), dy.contiguous(), eps)
      return dx, dscale.to(scale.dtype)
    dx, dscale = mesh_impl.slicewise(
        fn, *[lowering.tensors[t] for t in self.inputs])
    lowering.set_tensor_lowering(self.outputs[0], dx)
    lowering.set_tensor_lowering(self.outputs[1], dscale)


def sublayer_call_layer(x, layer_stack, context):
  """transformer.py:462-466."""
  x = sublayer_mask_padding(x, layer_stack, context)
  layer = context.current_layer
  with mtf.variable_scope(layer.__class__.__name__):
    return layer.call(context, x)


def sublayer_mask_padding(x, layer_stack, context):
  """Zeroes the padding positions (transformer.py:469-489); without a
  sequence_id tensor there is nothing to mask."""
  del layer_stack
  if isinstance(context.sequence_id, mtf.Tensor):
    return x * context.nonpadding
  return x


def sublayer_rms_norm(x, layer_stack, context, epsilon=1e-6, name="rms_norm"):
  """RMS normalisation with a learned scale `<name>/scale` [d_model]
  (transformer.py:493-516)."""
  del layer_stack
  model_dim = context.model.model_dim
  if context.model.ensemble_dims:
    raise NotImplementedError("ensembles are not implemented")
  with mtf.variable_scope(name):
    scale = mtf.get_variable(context.mesh, "scale", mtf.Shape([model_dim]),
                             initializer=mtf_layers.ones_initializer(),
                             dtype=context.variable_dtype)
  return RmsNormOperation(x, scale, epsilon, name=name).outputs[0]


def sublayer_legacy_rms_norm(x, layer_stack, context):
  """transformer.py:519-522."""
  return sublayer_rms_norm(x, layer_stack, context, name="layer_norm")


def sublayer_legacy_final_rms_norm(x, layer_stack, context):
  """transformer.py:525-528."""
  return sublayer_rms_norm(x, layer_stack, context, name="final_layer_norm")


def sublayer_residual(x, layer_stack, context):
  """transformer.py:584-587."""
  del layer_stack
  return x + context.current_layer_input


def sublayer_dropout(x, layer_stack, context, dropout_rate=0.0):
  """transformer.py:590-599: while training, one noise value per (batch
  entry, channel), shared by the positions of a sequence."""
  del layer_stack
  if context.train and dropout_rate > 0:
    return mtf.dropout(
        x, context.train, rate=dropout_rate,
        noise_shape=mtf.Shape(context.batch_dims + [context.model.model_dim]))
  return x


def sublayer_legacy_dropout(x, layer_stack, context):
  """transformer.py:627-636."""
  return sublayer_dropout(x, layer_stack, context,
                          dropout_rate=layer_stack.dropout_rate)


class LayerStack(TransformerLayer):
  """A stack of layers with residual connections and norms
  (transformer.py:314-457).  The default sublayers are those of the
  reference's defaults.gin."""

  def __init__(self, layers, sublayers_initial=None, sublayers_per_layer=None,
               sublayers_final=None, dropout_rate=None, norm_epsilon=None,
               recompute_grads=False):
    if recompute_grads:
      raise NotImplementedError("recompute_grads is not implemented")
    self._layers = layers
    self._sublayers_initial = sublayers_initial
    self._sublayers_per_layer = sublayers_per_layer
    self._sublayers_final = sublayers_final
    if (dropout_rate is not None) != (norm_epsilon is not None):
      raise ValueError(
          "LayerStack.dropout_rate and LayerStack.norm_epsilon should either "
          "be both not None (legacy mode) or both None (normal mode)")
    if dropout_rate is not None:
      # legacy mode, for old checkpoints' variable names (transformer.py:383-406)
      self.dropout_rate = dropout_rate
      self.norm_epsilon = norm_epsilon
      self._sublayers_initial = [sublayer_legacy_dropout]
      self._sublayers_per_layer = [sublayer_legacy_rms_norm,
                                   sublayer_call_layer,
                                   sublayer_legacy_dropout, sublayer_residual]
      self._sublayers_final = [sublayer_legacy_final_rms_norm,
                               sublayer_legacy_dropout]
    else:
      if self._sublayers_initial is None:
        self._sublayers_initial = [sublayer_dropout]
      if self._sublayers_per_layer is None:
        self._sublayers_per_layer = [sublayer_rms_norm, sublayer_call_layer,
                                     sublayer_dropout, sublayer_residual]
      if self._sublayers_final is None:
        self._sublayers_final = [sublayer_rms_norm, sublayer_dropout]

  def call(self, context, x):
    """transformer.py:408-428."""
    x = self._call_sublayers(self._sublayers_initial, x, context)
    context.layer_outputs.append(x)
    for lnum, layer in enumerate(self._layers):
      with mtf.variable_scope(layer.name or ""):
        x = self._layer_fn(x, layer, context)
      if lnum != len(self._layers) - 1:
        context.layer_outputs.append(x)
      context.layer_index += 1
    x = self._call_sublayers(self._sublayers_final, x, context)
    x = sublayer_mask_padding(x, self, context)
    context.layer_outputs.append(x)
    return x

  def _call_sublayers(self, sublayers, x, context):
    for s in sublayers:
      x = s(x, self, context)
    return x

  def _layer_fn(self, x, layer, context):
    context.current_layer = layer
    context.current_layer_input = x
    y = self._call_sublayers(self._sublayers_per_layer, x, context)
    if y.shape != x.shape:
      raise ValueError("Layer %s returned misshaped output x=%s y=%s"
                       % (layer.__class__.__name__, x, y))
    return y

  @property
  def num_layers(self):
    return len(self.layers)

  @property
  def layers(self):
    return self._layers


def _layer_spec(spec):
  """A class, or a list / tuple holding a class and optionally a name (str)
  and constructor arguments (dict), in any order."""
  if not isinstance(spec, (list, tuple)):
    return spec, None, {}
  cls, name, kwargs = None, None, {}
  for item in spec:
    if isinstance(item, str):
      name = item
    elif isinstance(item, dict):
      kwargs = item
    else:
      cls = item
  return cls, name, kwargs


def make_layer_stack(layers, num_layers=6, block_scope=True,
                     layer_stack_cls=LayerStack):
  """transformer.py:1876-1948: `layers` describes one block, repeated
  num_layers times.  Layer names are block_%03d/<name or layer_%03d> with
  block_scope, else <name> or layer_%03d counted over the whole stack."""
  built = []
  for block in range(num_layers):
    for n, spec in enumerate(layers):
      cls, name, kwargs = _layer_spec(spec)
      if block_scope:
        name = "block_%03d/%s" % (block, name or "layer_%03d" % n)
      elif not name:
        name = "layer_%03d" % len(built)
      layer = cls(**kwargs)
      layer.set_name(name)
      built.append(layer)
  return layer_stack_cls(built)


class Unitransformer(object):
  """The layer-stack call of the reference's Unitransformer
  (transformer.py:696-1075) on activations that are already embedded: model
  dims, the Context, and LayerStack.call under the model's name scope."""

  def __init__(self, layer_stack, d_model=1024, name="transformer",
               autoregressive=False, layout=None, mesh_shape=None,
               ensemble=None):
    if ensemble:
      raise NotImplementedError("ensembles are not implemented")
    self.layer_stack = layer_stack
    self.model_dim = mtf.Dimension("d_model", d_model)
    self.name = name
    self.autoregressive = autoregressive
    self.layout = layout
    self.mesh_shape = mesh_shape
    self.ensemble_dim = None

  @property
  def ensemble_dims(self):
    return []

  @property
  def fully_autoregressive(self):
    return self.autoregressive

  def call_layers(self, x, variable_dtype, mode=EVAL, num_microbatches=1,
                  sequence_id=None, position=None, states=None,
                  new_states=None, length_dim=None, reuse=None):
    """x [batch dims..., length, d_model] -> (y, losses).  The Context is the
    one _call_internal builds (transformer.py:1032-1062): read and write
    priorities are the position for an autoregressive model.

    Decoding, as sample_autoregressive drives it (transformer.py:1140-1248):
    mode "first_part" runs the known first part and appends every attention
    layer's keys and values to the list `new_states`; mode "incremental" takes
    x [batch dims..., d_model] (one position per batch entry), `position`
    [batch dims...] int32, the states of the previous call as `states`, the
    sequences' `length_dim`, and appends the updated states to `new_states`.
    The loop around it (sampling, stopping) stays with the caller.  `reuse`:
    take the variables an earlier call on this graph created (the default in
    "incremental" mode, as the reference's loop body does)."""
    if x.shape.dims[-1] != self.model_dim:
      raise ValueError("x %s does not end in %s" % (x.shape, self.model_dim))
    priority = POSITION if self.autoregressive else None
    losses = []
    if mode == INCREMENTAL:
      if length_dim is None:
        raise ValueError("incremental mode needs length_dim")
      batch_dims = x.shape.dims[:-1]
    else:
      batch_dims, length_dim = x.shape.dims[:-2], x.shape.dims[-2]
    context = Context(
        model=self, mesh=x.mesh, batch_dims=batch_dims,
        length_dim=length_dim, variable_dtype=variable_dtype, mode=mode,
        position=position, position_is_default=position is None,
        sequence_id=sequence_id, losses=losses,
        write_priority=priority, read_priority=priority,
        num_microbatches=num_microbatches, states=states,
        new_states=new_states)
    if reuse is None:
      reuse = mode == INCREMENTAL
    with mtf.variable_scope(self.name, reuse=reuse):
      y = self.layer_stack.call(context, x)
    return y, losses
