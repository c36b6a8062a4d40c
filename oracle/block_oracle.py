"""CPU restatement of the transformer block around the Mixture-of-Experts
layer: RMS norm, dense layers, multi-head self-attention and the LayerStack
that chains them with residual connections.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

NumPy float32 arithmetic with one rounding to the activation dtype per
reference op (float32 accumulation inside reductions and matmuls), as in
moe_oracle.  What pins each function (tests/test_block_oracle.py):

  rms_norm         float64 closed form; unit scale and constant rows give
                   x / |x| exactly representable cases
  dense            float64 matmul
  self_attention   float64 per-head softmax(q k^T + mask) v; causality (an
                   output does not change when later positions change); zero
                   queries give the running mean of the values
  layer_stack      zero output kernels reduce the stack to its final norm;
                   one layer by hand
  rms_norm_backward, dense_backward, attention_core_backward
                   float64 central differences of the forward formulas along
                   random directions, for every input; x-direction of the
                   norm's gradient vanishes when dy = x; the first causal
                   query's dq is zero
  dropout noise    (broadcast_dropout and the noise arguments) noise of ones
                   is the identity; float64 product; noise on the attention
                   weights equals noise on the values

PARITY UNPINNED against TensorFlow itself: the order of float32 accumulation
inside TF's reductions and matmuls, and for bfloat16 whether TF's reduce_sum
rounds partial sums (here: one rounding of a float32 sum).

Citations are to files under the reference tree (mesh_tensorflow/...).
"""

import math

import numpy as np

from oracle import moe_oracle as O

F32 = np.float32


def _r(a, act_dtype):
  return O.cast_act(np.asarray(a, F32), act_dtype)


def rms_norm(x, scale, act_dtype="float32", epsilon=1e-6):
  """sublayer_rms_norm (transformer/transformer.py:493-516):
  variance = reduce_mean(square(x), d_model); x * rsqrt(variance + eps) * scale.
  reduce_mean is reduce_sum times the Python float 1/M (ops.py:4807-4808);
  Python scalars enter an op rounded to the tensor dtype."""
  x = _r(x, act_dtype)
  scale = _r(scale, act_dtype)
  m = x.shape[-1]
  sq = _r(x * x, act_dtype)                                      # square
  total = _r(O.seq_sum(sq, axis=-1), act_dtype)                  # reduce_sum
  mean = _r(total * _r(F32(1.0 / m), act_dtype), act_dtype)      # * (1 / M)
  var = _r(mean + _r(F32(epsilon), act_dtype), act_dtype)        # + epsilon
  r = _r(F32(1.0) / np.sqrt(var, dtype=F32), act_dtype)          # rsqrt
  y = _r(x * r[..., None], act_dtype)                            # x * rsqrt
  return _r(y * scale, act_dtype)                                # * scale


def dense(x, w, act_dtype="float32", activation=None):
  """mtf.layers.dense without bias (layers.py:112-160): einsum over the last
  dim of x with float32 accumulation, result in the activation dtype, then
  the activation as its own op."""
  y = _r(np.matmul(_r(x, act_dtype), _r(w, act_dtype)), act_dtype)
  if activation == "relu":
    y = np.maximum(y, F32(0.0))
  elif activation not in (None, "linear"):
    raise ValueError("activation %r" % (activation,))
  return y


def broadcast_dropout(x, noise, axis, act_dtype="float32"):
  """mtf.dropout's product x * noise (ops.py:5872) with the noise broadcast
  over `axis` of x (a noise_shape without that dimension); `noise` is
  O.hidden_dropout_noise of the uniform draw."""
  return _r(_r(x, act_dtype) * np.expand_dims(_r(noise, act_dtype), axis),
            act_dtype)


def relative_position_bucket(relative_position, bidirectional=True,
                             num_buckets=32, max_distance=128):
  """_relative_position_bucket (transformer/transformer_layers.py:1000-1042):
  relative_position = memory position - query position (integers) -> bucket
  in [0, num_buckets).  Half of the buckets hold exact small distances, the
  other half grow logarithmically up to max_distance; with bidirectional the
  positive relative positions take the upper half of the range.  The
  logarithmic part is float32 arithmetic in the reference's op order
  (to_float(n) / max_exact, log, / the Python constant, * the integer, cast
  to int32 = truncation)."""
  rp = np.asarray(relative_position, np.int64)
  ret = np.zeros(rp.shape, np.int64)
  n = -rp
  if bidirectional:
    num_buckets //= 2
    ret = ret + (n < 0).astype(np.int64) * num_buckets
    n = np.abs(n)
  else:
    n = np.maximum(n, 0)
  max_exact = num_buckets // 2
  is_small = n < max_exact
  with np.errstate(divide="ignore"):
    ratio = np.log(n.astype(F32) / F32(max_exact)).astype(F32)
  scaled = (ratio / F32(math.log(max_distance / max_exact))).astype(F32) \
      * F32(num_buckets - max_exact)
  # (the small distances, whose logarithm is negative or -inf, are not taken)
  val_if_large = max_exact + np.where(is_small, 0, scaled).astype(np.int64)
  val_if_large = np.minimum(val_if_large, num_buckets - 1)
  return ret + np.where(is_small, n, val_if_large)


def relative_attention_bias(values, length, bidirectional, max_distance=128):
  """The bias SelfAttention.compute_bias adds for relative_attention_type
  "bias" / "bias_shared" (transformer_layers.py:317-352): values
  [H, num_buckets] gathered at the bucket of (memory position - query
  position) -> [1, H, L(query), L(key)]."""
  pos = np.arange(length)
  bucket = relative_position_bucket(pos[None, :] - pos[:, None], bidirectional,
                                    values.shape[-1], max_distance)
  return np.asarray(values, F32)[:, bucket][None]


def _visibility_bias(l, causal, sequence_id):
  """Sum of the attention biases of SelfAttention.compute_bias
  (transformer/transformer_layers.py:272-316) for the options built here, as
  [B or 1, 1, L(query), L(key)] float32: -1e9 where the key lies after the query
  (autoregressive, attention.py:830-842) and -1e9 where query and key carry
  different sequence ids (transformer_layers.py:303-316); the biases add."""
  bias = np.zeros((1, 1, l, l), F32)
  if causal:
    pos = np.arange(l)
    bias = bias + (pos[None, :] > pos[:, None]).astype(F32)[None, None] * F32(-1e9)
  if sequence_id is not None:
    sid = np.asarray(sequence_id)
    differ = (sid[:, :, None] != sid[:, None, :]).astype(F32)[:, None]
    bias = bias + differ * F32(-1e9)
  return bias


def self_attention(x, wq, wk, wv, wo, num_heads, causal, act_dtype="float32",
                   weights_noise=None, sequence_id=None, relative_values=None):
  """SelfAttention.call for the train / eval modes with the default options
  (transformer/transformer_layers.py:223-271) around attention.attention with
  float32 logits (transformer/attention.py:27-88).

  x [B, L, d_model]; wq, wk, wv [d_model, H*D]; wo [H*D, d_model].  q, k, v are
  activation-dtype tensors; logits = q . k in float32 (+ -1e9 where the key is
  not visible, attention.py:830-842; the bias is cast to the logits' dtype,
  :78-79); weights = mtf.softmax(logits) in float32, cast to the activation
  dtype; outputs = weights . v.  No 1/sqrt(d_kv) factor: it is folded into the
  initialiser of wq (attention.py:436-439).  weights_noise [B, H, L]: the
  dropout multiplier of the weights, one value per memory position, shared by
  the queries (attention.py:82-84 with dropout_broadcast_dims = [length]).
  """
  x = _r(x, act_dtype)
  b, l, _ = x.shape
  hd = wq.shape[1]
  d = hd // num_heads
  q = dense(x, wq, act_dtype).reshape(b, l, num_heads, d)
  k = dense(x, wk, act_dtype).reshape(b, l, num_heads, d)
  v = dense(x, wv, act_dtype).reshape(b, l, num_heads, d)
  logits = np.einsum("blhd,bmhd->bhlm", q, k).astype(F32)        # float32
  logits = (logits + _attention_bias(l, causal, sequence_id, relative_values,
                                     act_dtype)).astype(F32)
  weights = _r(O.softmax(logits), act_dtype)                     # cast to v's
  if weights_noise is not None:
    weights = broadcast_dropout(weights, weights_noise, 2, act_dtype)
  o = _r(np.einsum("bhlm,bmhd->blhd", weights, v), act_dtype)
  return dense(o.reshape(b, l, hd), wo, act_dtype)


def _attention_bias(l, causal, sequence_id, relative_values, act_dtype):
  """mtf.add_n of the biases (transformer_layers.py:352): the visibility
  biases plus, with relative_values [H, num_buckets], the relative attention
  bias (buckets of a bidirectional layout unless causal, :321-325); the sum is
  formed in the activation dtype and cast to the logits' float32
  (attention.py:78-79)."""
  bias = _visibility_bias(l, causal, sequence_id)
  if relative_values is None:
    return bias
  rel = relative_attention_bias(_r(relative_values, act_dtype), l, not causal)
  return _r(_r(bias, act_dtype) + rel, act_dtype).astype(F32)


def _attention_core(q, k, v, num_heads, causal, act_dtype, sequence_id=None,
                    relative_values=None):
  """attention.attention with float32 logits (attention.py:27-88) on
  [B, L, H*D] activation-dtype tensors -> [B, L, H*D]; sequence_id [B, L]
  integers or None."""
  b, l, hd = q.shape
  d = hd // num_heads
  q, k, v = (t.reshape(b, l, num_heads, d) for t in (q, k, v))
  logits = np.einsum("blhd,bmhd->bhlm", q, k).astype(F32)
  logits = (logits + _attention_bias(l, causal, sequence_id, relative_values,
                                     act_dtype)).astype(F32)
  weights = _r(O.softmax(logits), act_dtype)
  return _r(np.einsum("bhlm,bmhd->blhd", weights, v), act_dtype).reshape(b, l, hd)


def attention_incremental(q, k_new, v_new, k_cache, v_cache, position,
                          num_heads, act_dtype="float32", relative_values=None):
  """One decoding step of SelfAttention ("incremental" mode,
  transformer/transformer_layers.py:231-254 and :289-296): the step's key and
  value replace row position[b] of the recurrent states
  (k = old_k * (1 - one_hot) + k_new * one_hot), the query sees the memory
  positions m <= position[b] (read_priority >= write_priority), float32
  logits and softmax, weights cast to the activation dtype.

  q, k_new, v_new [B, H*D]; k_cache, v_cache [B, Lm, H*D]; position [B]
  integers.  relative_values [H, num_buckets]: the relative attention bias of
  memory position m against the step's position (compute_bias with
  context.position, transformer_layers.py:317-352; an autoregressive model's
  buckets are not bidirectional, :321).
  Returns (out [B, H*D], k [B, Lm, H*D], v [B, Lm, H*D])."""
  b, lm, hd = k_cache.shape
  d = hd // num_heads
  position = np.asarray(position).reshape(b)
  one_hot = _r((np.arange(lm)[None, :] == position[:, None]).astype(F32),
               act_dtype)[..., None]
  inv = _r(F32(1.0) - one_hot, act_dtype)
  k = _r(_r(_r(k_cache, act_dtype) * inv, act_dtype)
         + _r(_r(k_new, act_dtype)[:, None, :] * one_hot, act_dtype), act_dtype)
  v = _r(_r(_r(v_cache, act_dtype) * inv, act_dtype)
         + _r(_r(v_new, act_dtype)[:, None, :] * one_hot, act_dtype), act_dtype)
  q4 = _r(q, act_dtype).reshape(b, num_heads, d)
  k4, v4 = k.reshape(b, lm, num_heads, d), v.reshape(b, lm, num_heads, d)
  logits = np.einsum("bhd,bmhd->bhm", q4, k4).astype(F32)
  hidden = (np.arange(lm)[None, :] > position[:, None]).astype(F32)[:, None, :]
  bias = (hidden * F32(-1e9)).astype(F32)
  if relative_values is not None:
    values = _r(relative_values, act_dtype)
    bucket = relative_position_bucket(
        np.arange(lm)[None, :] - position[:, None], False, values.shape[-1])
    rel = values[:, bucket].transpose(1, 0, 2)                   # [B, H, Lm]
    bias = _r(_r(bias, act_dtype) + rel, act_dtype).astype(F32)
  logits = (logits + bias).astype(F32)
  weights = _r(O.softmax(logits), act_dtype)
  out = _r(np.einsum("bhm,bmhd->bhd", weights, v4), act_dtype)
  return out.reshape(b, hd), k, v


def experts_self_attention(x, w_gate, wi, q_wo, k_wo, wo, hparams, num_heads,
                           causal, act_dtype="float32", train=False,
                           num_microbatches=None):
  """ExpertsSelfAttention.call (transformer/transformer_layers.py:383-459 with
  attention.ExpertsAttentionParams, attention.py:594-692): a Mixture-of-Experts
  layer with moe_use_experts_attention projects x to [q, k] (two output
  kernels of the same experts, moe.py:514-522); q is scaled by d_kv ** -0.5
  (a Python scalar times a tensor: the scalar is rounded to the tensor's
  dtype); the keys are also the values; "o" projects the result back.

  hparams: an O.HParams for the experts layer (moe_use_experts_attention set).
  Returns (y [B, L, d_model], loss of the experts layer)."""
  x = _r(x, act_dtype)
  (q, k), loss, _ = O.moe_layer_v1(x, w_gate, wi, q_wo, hparams, train,
                                   act_dtype, k_wo=k_wo, dense=False,
                                   num_microbatches=num_microbatches)
  d = q.shape[-1] // num_heads
  q = _r(q * _r(F32(d ** -0.5), act_dtype), act_dtype)
  o = _attention_core(q, k, k, num_heads, causal, act_dtype)
  return dense(o, wo, act_dtype), loss


def dense_relu_dense(x, wi, wo, act_dtype="float32", hidden_noise=None):
  """DenseReluDense.call (transformer/transformer_layers.py:55-76);
  hidden_noise [B, d_ff]: the dropout multiplier of the hidden tensor, shared
  by the positions of a sequence (:67-69)."""
  h = dense(x, wi, act_dtype, "relu")
  if hidden_noise is not None:
    h = broadcast_dropout(h, hidden_noise, -2, act_dtype)
  return dense(h, wo, act_dtype)


def layer_stack(x, layers, final_scale, act_dtype="float32",
                autoregressive=False, train=False, initial_noise=None,
                final_noise=None, sequence_id=None):
  """LayerStack.call with the default sublayers (transformer/transformer.py:
  408-428 and the defaults quoted at :346-358): per layer
  dropout(x) first; per layer x + dropout(layer(rms_norm(x))); at the end
  dropout(rms_norm(x)).  Each dropout multiplies by a noise tensor
  [B, d_model] shared by the positions of a sequence (sublayer_dropout,
  transformer.py:590-599) and is skipped when its noise is None:
  initial_noise, final_noise, and per layer "sublayer_noise"; a layer's own
  dropout takes "weights_noise" (attention) or "hidden_noise"
  (dense_relu_dense).

  layers: list of dicts with "kind" in {"attention", "dense_relu_dense",
  "moe"}, "scale" (the layer's rms_norm scale) and the layer's weights:
    attention: wq, wk, wv, wo, num_heads; optional relative_values
      [heads, buckets], the layer's relative attention bias (the same array in
      every layer for relative_attention_type "bias_shared")
    dense_relu_dense: wi, wo
    moe: w_gate, wi, wo, hparams (an O.HParams); optional num_microbatches
    moe2d: w_outer, w_inner, wi, wo, hparams; optional num_microbatches
  sequence_id [B, L] integers (0 = padding) or None: every layer's input is
  multiplied by nonpadding = (sequence_id != 0) (sublayer_mask_padding inside
  sublayer_call_layer, transformer.py:462-489) and so is the stack's output
  (transformer.py:424), attention sees only keys of the query's own sequence,
  and the MoE layers get nonpadding (moe.py:117).
  Returns (y, losses) with one loss per MoE layer.
  """
  x = _r(x, act_dtype)
  nonpadding = None
  if sequence_id is not None:
    nonpadding = _r((np.asarray(sequence_id) != 0).astype(F32), act_dtype)
  if initial_noise is not None:
    x = broadcast_dropout(x, initial_noise, -2, act_dtype)
  losses = []
  for layer in layers:
    h = rms_norm(x, layer["scale"], act_dtype)
    if nonpadding is not None:
      h = _r(h * nonpadding[..., None], act_dtype)
    kind = layer["kind"]
    if kind == "attention":
      y = self_attention(h, layer["wq"], layer["wk"], layer["wv"], layer["wo"],
                         layer["num_heads"], autoregressive, act_dtype,
                         layer.get("weights_noise"), sequence_id,
                         layer.get("relative_values"))
    elif kind == "dense_relu_dense":
      y = dense_relu_dense(h, layer["wi"], layer["wo"], act_dtype,
                           layer.get("hidden_noise"))
    elif kind == "moe":
      y, loss, _ = O.moe_layer_v1(
          h, layer["w_gate"], layer["wi"], layer["wo"], layer["hparams"],
          train, act_dtype, nonpadding=nonpadding,
          num_microbatches=layer.get("num_microbatches"), dense=False)
      losses.append(loss)
    elif kind == "moe2d":
      # MoE2D.call -> transformer_moe_layer_v2 (transformer/moe.py:163-188)
      y, loss, _ = O.moe_layer_v2(
          h, layer["w_outer"], layer["w_inner"], layer["wi"], layer["wo"],
          layer["hparams"], train, act_dtype, nonpadding=nonpadding,
          num_microbatches=layer.get("num_microbatches"), dense=False)
      losses.append(loss)
    else:
      raise ValueError("layer kind %r" % (kind,))
    if layer.get("sublayer_noise") is not None:
      y = broadcast_dropout(y, layer["sublayer_noise"], -2, act_dtype)
    x = _r(y + x, act_dtype)                                     # residual
  y = rms_norm(x, final_scale, act_dtype)
  if final_noise is not None:
    y = broadcast_dropout(y, final_noise, -2, act_dtype)
  if nonpadding is not None:                       # transformer.py:424
    y = _r(y * nonpadding[..., None], act_dtype)
  return y, losses


# --- backward passes ----------------------------------------------------------
# The reference has no code of its own for these: mtf.gradients differentiates
# the einsum / reduce / cwise operations of the forward graph (ops.py:2846-2854
# and the gradient methods of the cwise operations).  They are restated as the
# derivatives of the forward formulas above, in float32 on the stored
# (activation-dtype) operands with one rounding per tensor that reaches memory,
# and pinned by float64 finite differences of the forward formulas.

def rms_norm_backward(x, scale, dy, act_dtype="float32", epsilon=1e-6):
  """(dx, dscale) of rms_norm: with r = rsqrt(mean(x^2) + eps), g = dy * scale:
  dx = r g - x r^3 mean(g x), dscale = sum over rows of dy x r."""
  x, scale, dy = _r(x, act_dtype), _r(scale, act_dtype), _r(dy, act_dtype)
  eps = _r(F32(epsilon), act_dtype)
  m = x.shape[-1]
  r = F32(1.0) / np.sqrt((x * x).sum(-1, keepdims=True, dtype=F32) / F32(m)
                         + eps, dtype=F32)
  g = dy * scale
  dot = (g * x).sum(-1, keepdims=True, dtype=F32) / F32(m)
  dx = g * r - x * (r * r * r * dot)
  dscale = (dy * x * r).reshape(-1, m).sum(0, dtype=F32)
  return _r(dx, act_dtype), _r(dscale, act_dtype)


def dense_backward(x, w, dy, act_dtype="float32", activation=None):
  """(dx, dw) of dense: dpre = dy (times (y > 0) after a relu), dx = dpre w^T,
  dw = x^T dpre over all leading dims."""
  x, w, dy = _r(x, act_dtype), _r(w, act_dtype), _r(dy, act_dtype)
  if activation == "relu":
    dy = _r(dy * (dense(x, w, act_dtype, "relu") > 0), act_dtype)
  elif activation not in (None, "linear"):
    raise ValueError("activation %r" % (activation,))
  k, n = w.shape
  dx = _r(np.matmul(dy, w.T), act_dtype)
  dw = _r(np.matmul(x.reshape(-1, k).T, dy.reshape(-1, n)), act_dtype)
  return dx, dw


def attention_core_backward(q, k, v, dout, num_heads, causal,
                            act_dtype="float32", sequence_id=None,
                            relative_values=None):
  """(dq, dk, dv) of _attention_core on [B, L, H*D] tensors: the weights as
  the forward pass rounds them; dweights = dout v^T, dv = weights^T dout,
  dlogits = weights (dweights - sum_k dweights weights), dq = dlogits k,
  dk = dlogits^T q; with relative_values [H, num_buckets] also their gradient
  as a fourth result."""
  b, l, hd = q.shape
  d = hd // num_heads
  q, k, v, dout = (_r(t, act_dtype).reshape(b, l, num_heads, d)
                   for t in (q, k, v, dout))
  logits = np.einsum("blhd,bmhd->bhlm", q, k).astype(F32)
  logits = (logits + _attention_bias(l, causal, sequence_id, relative_values,
                                     act_dtype)).astype(F32)
  weights = _r(O.softmax(logits), act_dtype)
  dweights = _r(np.einsum("blhd,bmhd->bhlm", dout, v), act_dtype)
  dv = _r(np.einsum("bhlm,blhd->bmhd", weights, dout), act_dtype)
  dot = (dweights * weights).sum(-1, keepdims=True, dtype=F32)
  dlogits = _r(weights * (dweights - dot), act_dtype)
  dq = _r(np.einsum("bhlm,bmhd->blhd", dlogits, k), act_dtype)
  dk = _r(np.einsum("bhlm,blhd->bmhd", dlogits, q), act_dtype)
  grads = tuple(t.reshape(b, l, hd) for t in (dq, dk, dv))
  if relative_values is None:
    return grads
  # the bias enters the logits once per batch entry: its gradient is dlogits
  # summed over the batch, scattered back to the buckets (gather's gradient)
  pos = np.arange(l)
  nb = np.asarray(relative_values).shape[-1]
  bucket = relative_position_bucket(pos[None, :] - pos[:, None], not causal, nb)
  dvalues = np.zeros((num_heads, nb), F32)
  per_head = dlogits.astype(F32).sum(0)                        # [H, L, L]
  for h in range(num_heads):
    np.add.at(dvalues[h], bucket.reshape(-1), per_head[h].reshape(-1))
  return grads + (_r(dvalues, act_dtype),)
