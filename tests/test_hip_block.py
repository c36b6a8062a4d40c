"""GPU parity of the transformer-block entry points (RMS norm, dense,
self-attention) and of a whole LayerStack with a MoE layer in it against
oracle/block_oracle.py."""

import os

import numpy as np
import pytest
import torch

import mesh_amd as mtf
from mesh_amd.transformer import moe
from mesh_amd.transformer import transformer
from mesh_amd.transformer import transformer_layers
from oracle import block_oracle as B
from oracle import moe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
  from mesh_amd import moe_hip
  moe_hip.load_library()
  return moe_hip


def _tol(act_dtype):
  return (dict(rtol=2e-2, atol=2e-2) if act_dtype == "bfloat16"
          else dict(rtol=1e-4, atol=2e-5))


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 7, 48), (2, 128, 1024), (1, 1, 8),
                                   (5, 33, 100)])
def test_rms_norm(hip, shape, act_dtype):
  rng = np.random.default_rng(sum(shape))
  x = O.cast_act(3 * rng.standard_normal(shape).astype(np.float32), act_dtype)
  scale = O.cast_act(1 + 0.2 * rng.standard_normal(shape[-1]).astype(np.float32),
                     act_dtype)
  got = H.to_np(hip.rms_norm(H.to_gpu(x, act_dtype), H.to_gpu(scale, act_dtype)))
  want = B.rms_norm(x, scale, act_dtype)
  if act_dtype == "float32":
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
  else:
    # the float32 sum is taken in another order: its bf16 rounding, and what
    # follows, can differ by one bf16 ulp
    np.testing.assert_allclose(got, want, rtol=1.6e-2, atol=1e-3)
    assert (got == want).mean() > 0.9


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(2, 9, 24, 40), (1, 300, 256, 512),
                                   (4, 64, 64, 128)])
def test_dense(hip, shape, act_dtype):
  b, l, k, n = shape
  rng = np.random.default_rng(sum(shape))
  x = O.cast_act(rng.standard_normal((b, l, k)).astype(np.float32), act_dtype)
  w = O.cast_act(H.normal_weights(rng, (k, n), k), act_dtype)
  wp = hip.pack_weights(H.to_gpu(w, act_dtype).reshape(1, k, n),
                        H.ACT_TORCH[act_dtype])
  for act in (None, "relu"):
    got = H.to_np(hip.dense(H.to_gpu(x, act_dtype), wp, act))
    np.testing.assert_allclose(got, B.dense(x, w, act_dtype, act),
                               **_tol(act_dtype))


ATT_CASES = [
    # B, L, heads, d_kv, d_model; bf16 with d_kv 64 / 128 runs the fused kernel
    (2, 12, 3, 4, 16), (1, 128, 4, 32, 64), (2, 200, 2, 64, 48),
    (1, 512, 8, 128, 256), (3, 64, 1, 16, 32), (2, 8, 2, 128, 32),
    (1, 72, 3, 64, 64), (2, 1000, 2, 128, 128), (1, 2048, 2, 128, 128),
    (3, 328, 1, 64, 32), (2, 13, 2, 12, 24),
]


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", ATT_CASES, ids=lambda c: "x".join(map(str, c)))
def test_self_attention(hip, case, causal, act_dtype):
  """The attention core (after the projections): q, k, v in, the outputs of
  the weights . v einsum out."""
  b, l, heads, d, m = case
  rng = np.random.default_rng(sum(case) + causal)
  x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
  hd = heads * d
  wq, wk, wv = (O.cast_act(H.normal_weights(rng, (m, hd), m), act_dtype)
                for _ in range(3))
  q, k, v = (B.dense(x, w, act_dtype) for w in (wq, wk, wv))
  got = H.to_np(hip.self_attention(
      H.to_gpu(q, act_dtype), H.to_gpu(k, act_dtype), H.to_gpu(v, act_dtype),
      heads, causal))
  want = _attention_core(q, k, v, heads, causal, act_dtype)
  tol = _tol(act_dtype)
  if act_dtype == "float32":
    tol = dict(rtol=1e-4, atol=1e-4)     # sums over up to 512 keys
  np.testing.assert_allclose(got, want, **tol)


def _attention_core(q, k, v, heads, causal, act_dtype):
  b, l, hd = q.shape
  d = hd // heads
  q4, k4, v4 = (t.reshape(b, l, heads, d) for t in (q, k, v))
  logits = np.einsum("blhd,bmhd->bhlm", q4, k4).astype(np.float32)
  if causal:
    pos = np.arange(l)
    logits = logits + (pos[None, :] > pos[:, None]).astype(np.float32) * \
        np.float32(-1e9)
  w = O.cast_act(O.softmax(logits), act_dtype)
  return O.cast_act(np.einsum("bhlm,bmhd->blhd", w, v4), act_dtype).reshape(
      b, l, hd)


def test_attention_core_helper_is_the_oracle():
  """_attention_core restates the middle of block_oracle.self_attention; with
  identity projections the two must agree exactly."""
  rng = np.random.default_rng(8)
  b, l, heads, d = 2, 10, 2, 4
  hd = heads * d
  x = rng.standard_normal((b, l, hd)).astype(np.float32)
  eye = np.eye(hd, dtype=np.float32)
  for causal in (False, True):
    np.testing.assert_array_equal(
        _attention_core(x, x, x, heads, causal, "float32"),
        B.self_attention(x, eye, eye, eye, eye, heads, causal))


def _packed_sequence_ids(rng, b, l, mean_len):
  """Packed sequences: ids 1, 2, ... over contiguous segments of random length,
  then a tail of padding (id 0) in every second batch entry."""
  ids = np.zeros((b, l), np.int32)
  for i in range(b):
    pos, sid = 0, 1
    stop = l if i % 2 == 0 else max(1, l - int(rng.integers(1, max(2, l // 4))))
    while pos < stop:
      n = int(rng.integers(1, 2 * mean_len))
      ids[i, pos:min(stop, pos + n)] = sid
      pos += n
      sid += 1
  return ids


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 40, 2, 16, 5), (2, 200, 2, 64, 37),
                                  (3, 328, 1, 128, 90), (2, 1000, 2, 128, 300),
                                  (1, 776, 2, 64, 20)],
                         ids=lambda c: "x".join(map(str, c)))
def test_self_attention_sequence_ids(hip, case, causal, act_dtype):
  """Packed / padded sequences (sequence ids, transformer_layers.py:303-316):
  forward and backward of the attention core against the oracle, through the
  fused kernels (bf16, d_kv 64 / 128) and the three-step form."""
  b, l, heads, d, mean_len = case
  rng = np.random.default_rng(sum(case) + causal)
  ids = _packed_sequence_ids(rng, b, l, mean_len)
  mk = lambda: O.cast_act(
      (rng.standard_normal((b, l, heads * d)) * 0.5).astype(np.float32),
      act_dtype)
  q, k, v, do = mk(), mk(), mk(), mk()
  g = lambda a: H.to_gpu(a, act_dtype)
  sid = torch.from_numpy(ids).cuda()
  got = H.to_np(hip.self_attention(g(q), g(k), g(v), heads, causal,
                                   sequence_id=sid))
  want = B._attention_core(q, k, v, heads, causal, act_dtype, sequence_id=ids)
  tol = _tol(act_dtype)
  if act_dtype == "float32":
    tol = dict(rtol=1e-4, atol=1e-4)
  np.testing.assert_allclose(got, want, **tol)
  # a token never sees another sequence: changing the other sequences' keys
  # and values leaves its output bits unchanged
  k2, v2 = k.copy(), v.copy()
  other = ids != ids[:, :1]
  k2[other] = O.cast_act(k2[other] * np.float32(-1.5) + np.float32(0.25), act_dtype)
  v2[other] = O.cast_act(v2[other] + np.float32(1.0), act_dtype)
  got2 = H.to_np(hip.self_attention(g(q), g(k2), g(v2), heads, causal,
                                    sequence_id=sid))
  np.testing.assert_array_equal(got2[~other], got[~other])
  want_b = B.attention_core_backward(q, k, v, do, heads, causal, act_dtype,
                                     sequence_id=ids)
  btol = dict(rtol=2e-4, atol=2e-4) if act_dtype == "float32" else dict(
      rtol=3e-2, atol=3e-2)
  for fused in ((None, False) if act_dtype == "bfloat16" else (None,)):
    got_b = hip.self_attention_backward(g(q), g(k), g(v), g(do), heads, causal,
                                        fused=fused, sequence_id=sid)
    for gt, wnt, name in zip(got_b, want_b, "qkv"):
      scale = max(1.0, float(np.abs(wnt).max()))
      np.testing.assert_allclose(H.to_np(gt), wnt, rtol=btol["rtol"],
                                 atol=btol["atol"] * scale,
                                 err_msg="d%s fused=%s" % (name, fused))


@pytest.mark.parametrize("causal", [True, False])
def test_attention_at_the_block_benchmark_shape(hip, causal):
  """The fused attention kernels at the (batch, head) shape of the benchmark
  block (L = 2048, 32 heads of 128; two batch entries instead of 32, the
  entries being independent) against the three-step pieces: the weights
  [B*H, L, L] of mesh_moe_attention_weights times v for the forward, the
  composed backward for the gradients; and causality as a property: keys and
  values after position p cannot change the outputs up to p."""
  b, l, heads, d = 2, 2048, 32, 128
  gen = torch.Generator(device="cuda").manual_seed(5)
  mk = lambda: (torch.randn((b, l, heads * d), generator=gen, device="cuda")
                * 0.3).to(torch.bfloat16)
  q, k, v, do = mk(), mk(), mk(), mk()
  out = hip.self_attention(q, k, v, heads, causal)
  w = hip.attention_weights(q, k, heads, causal)                 # [B*H, L, L]
  vh = v.reshape(b, l, heads, d).permute(0, 2, 1, 3).reshape(b * heads, l, d)
  want = torch.bmm(w.float(), vh.float()).reshape(b, heads, l, d).permute(
      0, 2, 1, 3).reshape(b, l, heads * d)
  torch.testing.assert_close(out.float(), want, rtol=2e-2, atol=2e-2)
  del w, want
  got = hip.self_attention_backward(q, k, v, do, heads, causal, fused=True)
  ref = hip.self_attention_backward(q, k, v, do, heads, causal, fused=False)
  for g_, r_, name in zip(got, ref, "qkv"):
    scale = max(1.0, float(r_.float().abs().max()))
    torch.testing.assert_close(g_.float(), r_.float(), rtol=3e-2,
                               atol=3e-2 * scale, msg="d" + name)
  if causal:
    p = 1237
    k2, v2 = k.clone(), v.clone()
    k2[:, p + 1:] = -k2[:, p + 1:]
    v2[:, p + 1:] = v2[:, p + 1:] + 1
    out2 = hip.self_attention(q, k2, v2, heads, causal)
    assert torch.equal(out2[:, :p + 1], out[:, :p + 1])
    assert not torch.equal(out2[:, p + 1:], out[:, p + 1:])


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [(2, 12, 2, 4), (3, 300, 4, 64), (2, 2048, 2, 128),
                                  (1, 77, 3, 24), (2, 40, 1, 320),
                                  (3, 2500, 2, 64)],
                         ids=lambda c: "x".join(map(str, c)))
def test_attention_decode(hip, case, act_dtype):
  """mesh_moe_attention_decode (one step of "incremental" mode) against the
  oracle: output and updated caches, positions from 0 to the last row."""
  b, lm, heads, d = case
  rng = np.random.default_rng(sum(case))
  hd = heads * d
  mk = lambda *shape: O.cast_act(
      (rng.standard_normal(shape) * 0.5).astype(np.float32), act_dtype)
  q, kn, vn = mk(b, hd), mk(b, hd), mk(b, hd)
  kc, vc = mk(b, lm, hd), mk(b, lm, hd)
  g = lambda a: H.to_gpu(a, act_dtype)
  for pos in ([0] * b, [lm - 1] * b, list(rng.integers(0, lm, size=b))):
    pos = np.asarray(pos, np.int32)
    want, want_k, want_v = B.attention_incremental(q, kn, vn, kc, vc, pos,
                                                   heads, act_dtype)
    kg, vg = g(kc), g(vc)
    got = hip.attention_decode(g(q), g(kn), g(vn), kg, vg,
                               torch.from_numpy(pos).cuda(), heads)
    tol = _tol(act_dtype)
    if act_dtype == "float32":
      tol = dict(rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(H.to_np(got), want, **tol)
    np.testing.assert_array_equal(H.to_np(kg), want_k)
    np.testing.assert_array_equal(H.to_np(vg), want_v)
    # with a relative attention bias against the step's position
    values = O.cast_act(rng.standard_normal((heads, 16)).astype(np.float32),
                        act_dtype)
    bucket = B.relative_position_bucket(np.arange(-(lm - 1), lm), False, 16)
    want_rel = B.attention_incremental(q, kn, vn, kc, vc, pos, heads, act_dtype,
                                       relative_values=values)[0]
    got_rel = hip.attention_decode(
        g(q), g(kn), g(vn), g(kc), g(vc), torch.from_numpy(pos).cuda(), heads,
        relative_bias=(g(values),
                       torch.from_numpy(bucket.astype(np.int32)).cuda()))
    np.testing.assert_allclose(H.to_np(got_rel), want_rel, **tol)
    if lm > 1 and pos.max() > 0:
      assert np.abs(want_rel - want).max() > 1e-3


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 40, 2, 16, 8), (2, 200, 3, 64, 32),
                                  (1, 328, 2, 128, 32), (1, 1024, 2, 64, 32),
                                  (2, 576, 1, 128, 8)],
                         ids=lambda c: "x".join(map(str, c)))
def test_self_attention_relative_bias(hip, case, causal, act_dtype):
  """The relative attention bias (transformer_layers.py:317-352): forward,
  (dq, dk, dv) and the gradient of the bias values against the oracle, with and
  without sequence ids.  bf16 with d_kv 64 or 128 runs the fused kernels
  (forward and backward), whose composed counterpart (fused=False) is checked
  as well; everything else the three-step form."""
  b, l, heads, d, nb = case
  rng = np.random.default_rng(sum(case) + causal)
  mk = lambda: O.cast_act(
      (rng.standard_normal((b, l, heads * d)) * 0.5).astype(np.float32),
      act_dtype)
  q, k, v, do = mk(), mk(), mk(), mk()
  values = O.cast_act(rng.standard_normal((heads, nb)).astype(np.float32),
                      act_dtype)
  pos = np.arange(-(l - 1), l)
  bucket = B.relative_position_bucket(pos, not causal, nb).astype(np.int32)
  g = lambda a: H.to_gpu(a, act_dtype)
  rel = (g(values), torch.from_numpy(bucket).cuda())
  for ids in (None, _packed_sequence_ids(rng, b, l, max(4, l // 3))):
    sid = None if ids is None else torch.from_numpy(ids).cuda()
    got = H.to_np(hip.self_attention(g(q), g(k), g(v), heads, causal,
                                     sequence_id=sid, relative_bias=rel))
    want = B._attention_core(q, k, v, heads, causal, act_dtype, sequence_id=ids,
                             relative_values=values)
    tol = _tol(act_dtype)
    if act_dtype == "float32":
      tol = dict(rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(got, want, **tol)
    got_b = hip.self_attention_backward(g(q), g(k), g(v), g(do), heads, causal,
                                        sequence_id=sid, relative_bias=rel)
    want_b = B.attention_core_backward(q, k, v, do, heads, causal, act_dtype,
                                       sequence_id=ids, relative_values=values)
    btol = dict(rtol=2e-4, atol=2e-4) if act_dtype == "float32" else dict(
        rtol=3e-2, atol=3e-2)
    runs = [("", got_b)]
    if act_dtype == "bfloat16" and d in (64, 128):
      runs.append(("composed ", hip.self_attention_backward(
          g(q), g(k), g(v), g(do), heads, causal, fused=False, sequence_id=sid,
          relative_bias=rel)))
    for label, grads in runs:
      assert len(grads) == 4
      for gt, wnt, name in zip(grads, want_b, ("dq", "dk", "dv", "dvalues")):
        scale = max(1.0, float(np.abs(wnt).max()))
        np.testing.assert_allclose(H.to_np(gt), wnt, rtol=btol["rtol"],
                                   atol=btol["atol"] * scale,
                                   err_msg=label + name)
  # not the same as no bias
  plain = H.to_np(hip.self_attention(g(q), g(k), g(v), heads, causal))
  assert np.abs(plain - got).max() > 1e-2


def test_self_attention_rejections(hip):
  q = torch.zeros((1, 12, 16), dtype=torch.bfloat16, device="cuda")
  with pytest.raises(hip.MoeHipError, match="not divisible"):
    hip.self_attention(q, q, q, 3, True)


def _build_stack(rng, m, e, hdim, heads, d, group):
  def n(*shape):
    return H.normal_weights(rng, shape, shape[-2])
  def scale():
    return (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  att = lambda: dict(kind="attention", num_heads=heads, wq=n(m, heads * d),
                     wk=n(m, heads * d), wv=n(m, heads * d),
                     wo=n(heads * d, m), scale=scale())
  hp_kw = dict(moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
               moe_second_policy_eval="all", moe_second_policy_train="all",
               moe_capacity_factor_eval=2.0)
  moe_l = dict(kind="moe", w_gate=n(m, e), wi=n(e, m, hdim), wo=n(e, hdim, m),
               hparams=O.default_hparams(**hp_kw), scale=scale())
  ffn = dict(kind="dense_relu_dense", wi=n(m, hdim), wo=n(hdim, m),
             scale=scale())
  return [att(), moe_l, att(), ffn], scale()


def _run_stack(x, layers, final, act_dtype, heads, d, e, hdim, group,
               autoregressive, sequence_id=None, with_gradients=False):
  dt = H.ACT_TORCH[act_dtype]
  b, l, m = x.shape
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention,
        dict(num_heads=heads, key_value_size=d)),
       (moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                        second_policy_train="all", second_policy_eval="all",
                        capacity_factor_eval=2.0)),
       (transformer_layers.SelfAttention,
        dict(num_heads=heads, key_value_size=d)),
       (transformer_layers.DenseReluDense, dict(hidden_size=hdim))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=autoregressive)
  ids = None
  if sequence_id is not None:
    ids = mtf.import_tf_tensor(mesh, torch.from_numpy(sequence_id),
                               mtf.Shape(dims[:2]))
  y, losses = model.call_layers(
      xt, mtf.VariableDType(torch.float32, torch.float32, dt), mode="eval",
      sequence_id=ids)
  grads = []
  if with_gradients:
    grads = mtf.gradients([y] + list(losses),
                          [xt] + [v.outputs[0] for v in graph.trainable_variables])
  init = {"decoder/rms_norm/scale": final}
  for i, layer in enumerate(layers):
    p = "decoder/layer_%03d/" % i
    init[p + "rms_norm/scale"] = layer["scale"]
    if layer["kind"] == "attention":
      for k in "qkvo":
        init[p + "SelfAttention/" + k] = layer["w" + k]
    elif layer["kind"] == "moe":
      init[p + "MoE1D/top_2_gating/kernel"] = layer["w_gate"]
      init[p + "MoE1D/wi/kernel"] = layer["wi"]
      init[p + "MoE1D/wo/kernel"] = layer["wo"]
    else:
      init[p + "DenseReluDense/wi/kernel"] = layer["wi"]
      init[p + "DenseReluDense/wo/kernel"] = layer["wo"]
  assert sorted(init) == sorted(v.name for v in graph.all_variables)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  out = H.to_np(lowering.export_to_tf_tensor(y))
  loss = [float(H.to_np(lowering.export_to_tf_tensor(t))) for t in losses]
  if with_gradients:
    return out, loss, [H.to_np(lowering.export_to_tf_tensor(g)) for g in grads]
  return out, loss


@pytest.mark.parametrize("autoregressive", [True, False])
def test_layer_stack_float32(autoregressive):
  """Attention, MoE1D, attention, DenseReluDense (the block of
  transformer/gin/models/lm_moe.gin) through the graph API against the
  oracle."""
  b, l, m, e, hdim, heads, d, group = 2, 64, 64, 4, 96, 4, 16, 32
  rng = np.random.default_rng(21)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  got, got_loss = _run_stack(x, layers, final, "float32", heads, d, e, hdim,
                             group, autoregressive)
  want, want_loss = B.layer_stack(x, layers, final, "float32", autoregressive)
  np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)


@pytest.mark.parametrize("autoregressive", [True, False])
def test_layer_stack_packed_sequences(autoregressive):
  """The same block on packed, padded rows (Context.sequence_id): every layer's
  input is multiplied by nonpadding, attention stays inside a sequence, the
  experts' router gets nonpadding as importance -- against the oracle; the
  gradient graph of the packed block lowers and is finite."""
  b, l, m, e, hdim, heads, d, group = 2, 64, 64, 4, 96, 4, 16, 32
  rng = np.random.default_rng(23)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  ids = np.array([[1] * 20 + [2] * 30 + [3] * 9 + [0] * 5,
                  [4] * 41 + [5] * 23], np.int32)
  got, got_loss, grads = _run_stack(x, layers, final, "float32", heads, d, e,
                                    hdim, group, autoregressive,
                                    sequence_id=ids, with_gradients=True)
  want, want_loss = B.layer_stack(x, layers, final, "float32", autoregressive,
                                  sequence_id=ids)
  np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)
  # not the same as ignoring the ids
  plain, _ = B.layer_stack(x, layers, final, "float32", autoregressive)
  assert np.abs(plain - want).max() > 1e-2
  assert all(np.isfinite(g).all() for g in grads)
  # the stack's output is zero at the padding positions, and with it the
  # gradient of their inputs (they only reach other padding positions)
  assert not got[0, -5:].any() and not grads[0][0, -5:].any()


@pytest.mark.parametrize("autoregressive", [True, False])
@pytest.mark.parametrize("kind", ["bias", "bias_shared"])
def test_layer_stack_relative_attention_bias(kind, autoregressive):
  """SelfAttention(relative_attention_type="bias" / "bias_shared") in a stack
  (transformer_layers.py:317-352): "bias" gives every attention layer its own
  variable "relative_attention_bias" [heads, buckets]; "bias_shared" creates
  it in the first one and reuses it.  Output against the oracle; the gradient
  of the variables against the oracle's backward passes chained by hand
  (shared: the two layers' contributions add up)."""
  b, l, m, heads, d, nb = 2, 48, 64, 4, 16, 32
  rng = np.random.default_rng(71)
  layers, final = _build_stack(rng, m, 4, 96, heads, d, 32)
  a0, a1 = layers[0], layers[2]
  a0["relative_values"] = rng.standard_normal((heads, nb)).astype(np.float32)
  a1["relative_values"] = (a0["relative_values"] if kind == "bias_shared" else
                           rng.standard_normal((heads, nb)).astype(np.float32))
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  dy = rng.standard_normal((b, l, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy), mtf.Shape(dims))
  att_kw = dict(num_heads=heads, key_value_size=d, relative_attention_type=kind,
                relative_attention_num_buckets=nb)
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention, att_kw),
       (transformer_layers.SelfAttention, att_kw)],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=autoregressive)
  y, _ = model.call_layers(xt, mtf.VariableDType(torch.float32), mode="eval")
  init = {"decoder/rms_norm/scale": final}
  for i, att in enumerate((a0, a1)):
    p = "decoder/layer_%03d/" % i
    init[p + "rms_norm/scale"] = att["scale"]
    for c in "qkvo":
      init[p + "SelfAttention/" + c] = att["w" + c]
    if i == 0 or kind == "bias":
      init[p + "SelfAttention/relative_attention_bias"] = att["relative_values"]
  variables = {v.name: v for v in graph.all_variables}
  assert sorted(variables) == sorted(init)
  rel_names = sorted(n for n in init if n.endswith("relative_attention_bias"))
  grads = mtf.gradients([y], [variables[n].outputs[0] for n in rel_names], [dyt])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = H.to_np(lowering.export_to_tf_tensor(y))
  want, _ = B.layer_stack(x, [a0, a1], final, "float32", autoregressive)
  np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
  plain, _ = B.layer_stack(
      x, [{k: v for k, v in a.items() if k != "relative_values"}
          for a in (a0, a1)], final, "float32", autoregressive)
  assert np.abs(plain - want).max() > 1e-2
  # backward by hand: final norm <- layer 1 <- layer 0, keeping each
  # attention's gradient of its bias values
  xs, cores = [x], []
  for att in (a0, a1):
    h = B.rms_norm(xs[-1], att["scale"])
    q, k, v = (B.dense(h, att["w" + c]) for c in "qkv")
    o = B._attention_core(q, k, v, heads, autoregressive, "float32",
                          relative_values=att["relative_values"])
    cores.append((q, k, v, o))
    xs.append(xs[-1] + B.dense(o, att["wo"]))
  dx, _ = B.rms_norm_backward(xs[2], final, dy)
  dvalues = []
  for att, (q, k, v, o), x_in in reversed(list(zip((a0, a1), cores, xs[:2]))):
    do, _ = B.dense_backward(o, att["wo"], dx)
    dq, dk, dv, dval = B.attention_core_backward(
        q, k, v, do, heads, autoregressive,
        relative_values=att["relative_values"])
    dvalues.insert(0, dval)
    h = B.rms_norm(x_in, att["scale"])
    dh = sum(B.dense_backward(h, att["w" + c], g)[0]
             for c, g in zip("qkv", (dq, dk, dv)))
    dx = dx + B.rms_norm_backward(x_in, att["scale"], dh)[0]
  want_grads = [dvalues[0] + dvalues[1]] if kind == "bias_shared" else dvalues
  assert len(grads) == len(want_grads)
  for g, w in zip(grads, want_grads):
    g = H.to_np(lowering.export_to_tf_tensor(g))
    assert np.abs(w).max() > 1e-2
    np.testing.assert_allclose(g, w, rtol=1e-3, atol=1e-3 * np.abs(w).max())


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_captured_stack_with_relative_bias_replays_match_eager(act_dtype):
  """A stack with relative attention bias recorded into a HIP graph: the
  bucket table of the length is already on the device when the recording
  starts (a pageable host-to-device copy could not be recorded), and every
  replay on new tokens gives what the eager run gives."""
  b, l, m, heads, d, nb = 2, 128, 128, 2, 64, 32
  dt = H.ACT_TORCH[act_dtype]
  gen = torch.Generator().manual_seed(5)
  xs = [torch.randn((b, l, m), generator=gen).to(dt) for _ in range(3)]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, xs[0], mtf.Shape(dims))
  att_kw = dict(num_heads=heads, key_value_size=d,
                relative_attention_type="bias",
                relative_attention_num_buckets=nb)
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention, att_kw),
       (transformer_layers.DenseReluDense, dict(hidden_size=256))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=True)
  y, _ = model.call_layers(xt, mtf.VariableDType(dt, dt, dt), mode="eval")
  torch.manual_seed(11)
  lowering = mtf.Lowering(
      graph, {mesh: mtf.HipMeshImpl()},
      initial_values={
          "decoder/layer_000/SelfAttention/relative_attention_bias":
              torch.randn((heads, nb), generator=gen).numpy()})
  from mesh_amd.transformer import attention
  before = dict(attention._BUCKET_TABLES)
  assert any(k[0] == l and k[2] == nb for k in before)
  step = lowering.capture()
  # the recording made no new table and re-used the one it found
  assert set(attention._BUCKET_TABLES) == set(before)
  assert all(attention._BUCKET_TABLES[k] is before[k] for k in before)
  for i in (1, 2, 0, 1):
    xv = xs[i].cuda()
    lowering.run({xt: xv})
    eager = lowering.export_to_tf_tensor(y).clone()
    torch.cuda.synchronize()
    step.replay({xt: xv})
    torch.cuda.synchronize()
    assert torch.equal(lowering.export_to_tf_tensor(y), eager), i
  assert bool(torch.isfinite(eager.float()).all()) and float(eager.float().abs().max()) > 0


@pytest.mark.parametrize("relative,shared_kv", [(None, False),
                                                ("bias_shared", False),
                                                ("bias_shared", True)])
@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_decoding_modes_match_the_full_forward(act_dtype, relative, shared_kv):
  """Decoding as Unitransformer.sample_autoregressive drives it
  (transformer.py:1140-1248): "first_part" over a row whose positions from p0
  on are unknown (zeros) records every attention layer's keys and values; one
  "incremental" call per position p >= p0 takes the token of that position, the
  states and position [batch], and must give what the full forward gives at p
  (teacher forcing).  The experts' capacity is ample in both runs, so no token
  is dropped in either.  With relative = "bias_shared" the attention layers add
  the first layer's relative attention bias in all three modes."""
  b, l, m, e, hdim, heads, d, group, p0 = 2, 24, 64, 4, 96, 4, 16, 32, 17
  dt = H.ACT_TORCH[act_dtype]
  rng = np.random.default_rng(61)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  batch, length, model_dim = (mtf.Dimension("batch", b), mtf.Dimension("length", l),
                              mtf.Dimension("d_model", m))
  if shared_kv:          # one kernel for keys and values, one state per layer
    for layer in layers:
      if layer["kind"] == "attention":
        layer["wv"] = layer["wk"]
  att_kw = dict(num_heads=heads, key_value_size=d, shared_kv=shared_kv,
                relative_attention_type=relative,
                relative_attention_num_buckets=8)
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention, att_kw),
       (moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                        second_policy_train="all", second_policy_eval="all",
                        capacity_factor_eval=float(e))),
       (transformer_layers.SelfAttention, att_kw),
       (transformer_layers.DenseReluDense, dict(hidden_size=hdim))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=True)
  vdt = mtf.VariableDType(torch.float32, torch.float32, dt)
  to_t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dt)
  full_in = mtf.import_tf_tensor(mesh, to_t(x), mtf.Shape([batch, length, model_dim]))
  y_full, _ = model.call_layers(full_in, vdt, mode="eval")
  first = x.copy()
  first[:, p0:] = 0
  first_in = mtf.import_tf_tensor(mesh, to_t(first),
                                  mtf.Shape([batch, length, model_dim]))
  states = []
  y_first, _ = model.call_layers(first_in, vdt, mode="first_part",
                                 new_states=states, reuse=True)
  assert len(states) == (2 if shared_kv else 4)
  assert all(t.shape.dimension_names == ["batch", "memory_length", "heads"]
             for t in states)
  steps = []
  for p in range(p0, l):
    tok = mtf.import_tf_tensor(mesh, to_t(x[:, p]), mtf.Shape([batch, model_dim]))
    pos = mtf.import_tf_tensor(mesh, torch.full((b,), p, dtype=torch.int32),
                               mtf.Shape([batch]))
    new_states = []
    y_p, _ = model.call_layers(tok, vdt, mode="incremental", position=pos,
                               states=states, new_states=new_states,
                               length_dim=length)
    assert y_p.shape.dimension_names == ["batch", "d_model"]
    steps.append(y_p)
    states = new_states
  init = {"decoder/rms_norm/scale": final}
  for i, layer in enumerate(layers):
    prefix = "decoder/layer_%03d/" % i
    init[prefix + "rms_norm/scale"] = layer["scale"]
    if layer["kind"] == "attention":
      for c in ("q", "kv", "o") if shared_kv else "qkvo":
        init[prefix + "SelfAttention/" + c] = layer["w" + c[0]]
    elif layer["kind"] == "moe":
      init[prefix + "MoE1D/top_2_gating/kernel"] = layer["w_gate"]
      init[prefix + "MoE1D/wi/kernel"] = layer["wi"]
      init[prefix + "MoE1D/wo/kernel"] = layer["wo"]
    else:
      init[prefix + "DenseReluDense/wi/kernel"] = layer["wi"]
      init[prefix + "DenseReluDense/wo/kernel"] = layer["wo"]
  if relative:
    init["decoder/layer_000/SelfAttention/relative_attention_bias"] = (
        rng.standard_normal((heads, 8)).astype(np.float32))
  assert sorted(init) == sorted(v.name for v in graph.all_variables)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  want = H.to_np(lowering.export_to_tf_tensor(y_full))
  if act_dtype == "float32":
    # the full forward is the oracle's (same ample capacity for the experts)
    layers[1]["hparams"] = O.default_hparams(
        moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
        moe_second_policy_eval="all", moe_second_policy_train="all",
        moe_capacity_factor_eval=float(e))
    plain, _ = B.layer_stack(x, layers, final, act_dtype, True)
    if relative:   # the bias matters: the oracle without it is somewhere else
      assert np.abs(plain - want).max() > 5e-2
      for layer in layers:
        if layer["kind"] == "attention":
          layer["relative_values"] = init[
              "decoder/layer_000/SelfAttention/relative_attention_bias"]
    oracle_full, _ = B.layer_stack(x, layers, final, act_dtype, True)
    np.testing.assert_allclose(want, oracle_full, rtol=2e-4, atol=2e-4)
  got_first = H.to_np(lowering.export_to_tf_tensor(y_first))
  tol = dict(rtol=2e-4, atol=2e-4) if act_dtype == "float32" else dict(
      rtol=5e-2, atol=5e-2)
  # the known first part sees only itself (autoregressive)
  np.testing.assert_allclose(got_first[:, :p0], want[:, :p0], **tol)
  for p, y_p in zip(range(p0, l), steps):
    got = H.to_np(lowering.export_to_tf_tensor(y_p))
    if act_dtype == "float32":
      np.testing.assert_allclose(got, want[:, p], err_msg="position %d" % p, **tol)
    else:
      # a token whose two best experts nearly tie can be routed differently
      # when its router input differs by a bf16 ulp between the two runs
      ok = np.isclose(got, want[:, p], **tol).all(axis=-1)
      assert ok.mean() >= 0.5, (p, ok)
  # the final states hold the keys of the full row: layer 0's keys are a
  # projection of its normed input, the same in both runs
  k_full = [op for op in graph.operations
            if type(op).__name__ == "SelfAttentionOperation"][0].inputs[1]
  np.testing.assert_allclose(
      H.to_np(lowering.export_to_tf_tensor(states[0])),
      H.to_np(lowering.export_to_tf_tensor(k_full)), **tol)


@pytest.mark.parametrize("train", [False, True])
def test_layer_stack_with_moe2d(train):
  """MoE2D.call (transformer/moe.py:163-188) inside a LayerStack: the
  hierarchical layer behind rms_norm and the residual, followed by a
  DenseReluDense, against the oracle's transformer_moe_layer_v2; the capacity
  factor differs between train and eval mode, so both modes are run."""
  b, l, m, hdim, xe, ye, group = 2, 96, 32, 48, 3, 4, 48
  rng = np.random.default_rng(27)
  n = lambda *shape: H.normal_weights(rng, shape, shape[-2])
  scale = lambda: (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  kw = dict(expert_x=xe, expert_y=ye, hidden_size=hdim, group_size=group,
            capacity_factor_train=1.25, capacity_factor_eval=2.0,
            capacity_factor_second_level=1.5, second_policy_train="all",
            second_policy_eval="all")
  ohp = O.default_hparams(
      moe_num_experts=[xe, ye], moe_hidden_size=hdim, moe_group_size=group,
      moe_capacity_factor_train=1.25, moe_capacity_factor_eval=2.0,
      moe_capacity_factor_second_level=1.5, moe_second_policy_train="all",
      moe_second_policy_eval="all", moe_min_expert_capacity=4)
  layers = [dict(kind="moe2d", w_outer=n(m, xe), w_inner=n(xe, m, ye),
                 wi=n(ye, xe, m, hdim), wo=n(ye, xe, hdim, m), hparams=ohp,
                 scale=scale()),
            dict(kind="dense_relu_dense", wi=n(m, hdim), wo=n(hdim, m),
                 scale=scale())]
  final = scale()
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(moe.MoE2D, kw), (transformer_layers.DenseReluDense,
                         dict(hidden_size=hdim, dropout_rate=0.0))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=False)
  y, losses = model.call_layers(
      xt, mtf.VariableDType(torch.float32, torch.float32, torch.float32),
      mode="train" if train else "eval")
  p0, p1 = "decoder/layer_000/", "decoder/layer_001/"
  init = {"decoder/rms_norm/scale": final,
          p0 + "rms_norm/scale": layers[0]["scale"],
          p0 + "MoE2D/outer_gating/kernel": layers[0]["w_outer"],
          p0 + "MoE2D/inner_gating/kernel": layers[0]["w_inner"],
          p0 + "MoE2D/wi/kernel": layers[0]["wi"],
          p0 + "MoE2D/wo/kernel": layers[0]["wo"],
          p1 + "rms_norm/scale": layers[1]["scale"],
          p1 + "DenseReluDense/wi/kernel": layers[1]["wi"],
          p1 + "DenseReluDense/wo/kernel": layers[1]["wo"]}
  assert sorted(init) == sorted(v.name for v in graph.all_variables)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = H.to_np(lowering.export_to_tf_tensor(y))
  got_loss = [float(H.to_np(lowering.export_to_tf_tensor(t))) for t in losses]
  want, want_loss = B.layer_stack(x, layers, final, "float32", False,
                                  train=train)
  assert len(got_loss) == 1
  np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)


def test_layer_stack_bfloat16():
  """In bfloat16 the tokens that reach the router differ by a bf16 ulp here and
  there between the two implementations (different float32 summation orders
  upstream), so a few tokens whose two best experts are nearly tied are routed
  differently; the comparison is per token and asks for 95 % of them."""
  b, l, m, e, hdim, heads, d, group = 2, 128, 128, 4, 256, 4, 32, 64
  rng = np.random.default_rng(22)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = O.round_bf16(rng.standard_normal((b, l, m)).astype(np.float32))
  got, got_loss = _run_stack(x, layers, final, "bfloat16", heads, d, e, hdim,
                             group, True)
  want, want_loss = B.layer_stack(x, layers, final, "bfloat16", True)
  assert np.isfinite(got).all()
  ok = np.isclose(got, want, rtol=5e-2, atol=5e-2).all(axis=-1)
  assert ok.mean() >= 0.95, ok.mean()
  np.testing.assert_allclose(got_loss, want_loss, rtol=2e-2)


def test_checkpoint_round_trip(tmp_path):
  """Variables saved by name to an .npz archive, or to a tensor bundle, and
  restored into a freshly initialised lowering of the same graph reproduce the
  outputs; a filter
  restores only the matching names; a wrong shape raises."""
  from mesh_amd import checkpoint
  b, l, m, e, hdim, heads, d, group = 1, 32, 32, 4, 48, 2, 16, 32
  rng = np.random.default_rng(31)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = rng.standard_normal((b, l, m)).astype(np.float32)

  def build():
    graph = mtf.Graph()
    mesh = mtf.Mesh(graph, "mesh")
    dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
            mtf.Dimension("d_model", m)]
    xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
    stack = transformer.make_layer_stack(
        [(transformer_layers.SelfAttention,
          dict(num_heads=heads, key_value_size=d)),
         (moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                          second_policy_train="all", second_policy_eval="all")),
         (transformer_layers.DenseReluDense, dict(hidden_size=hdim))],
        num_layers=1, block_scope=False)
    model = transformer.Unitransformer(stack, d_model=m, name="decoder")
    y, _ = model.call_layers(xt, mtf.VariableDType(torch.float32))
    lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()})
    return lowering, y

  low_a, y_a = build()                       # random initial values
  out_a = H.to_np(low_a.export_to_tf_tensor(y_a))
  path = str(tmp_path / "model.npz")
  saved = checkpoint.save_variables(low_a, path)
  assert "decoder/layer_001/MoE1D/top_2_gating/kernel" in saved
  low_b, y_b = build()                       # other random values
  assert np.abs(H.to_np(low_b.export_to_tf_tensor(y_b)) - out_a).max() > 1e-3
  report = checkpoint.restore_variables(low_b, path)
  assert sorted(report.restored) == sorted(saved)
  assert not report.in_graph_not_in_checkpoint
  low_b.run()
  np.testing.assert_array_equal(H.to_np(low_b.export_to_tf_tensor(y_b)), out_a)
  # the same through a TensorFlow tensor bundle: by prefix, then by directory
  prefix = str(tmp_path / "run" / "model.ckpt-100")
  checkpoint.save_variables(low_a, prefix)
  assert os.path.exists(prefix + ".index")
  assert os.path.exists(prefix + ".data-00000-of-00001")
  for source in (prefix, str(tmp_path / "run")):
    low_d, y_d = build()
    report = checkpoint.restore_variables(low_d, source)
    assert sorted(report.restored) == sorted(saved)
    low_d.run()
    np.testing.assert_array_equal(H.to_np(low_d.export_to_tf_tensor(y_d)),
                                  out_a)
  with pytest.raises(ValueError, match="no checkpoint state"):
    checkpoint.restore_variables(low_b, str(tmp_path))
  low_c, _ = build()
  report = checkpoint.restore_variables(low_c, saved, variable_filter="MoE1D")
  assert sorted(report.restored) == sorted(n for n in saved if "MoE1D" in n)
  bad = dict(saved)
  bad["decoder/rms_norm/scale"] = np.ones(m + 1, np.float32)
  with pytest.raises(ValueError, match="has shape"):
    checkpoint.restore_variables(low_c, bad)


def test_dense_rows_beyond_2_to_the_30_elements(hip):
  """A dense layer whose input has more than 2^30 elements (98304 tokens x
  16384 channels): the direct-to-LDS kernels address rows with 32-bit element
  offsets, which must hold up to 2^31.  Checked on the first and last rows
  against a float32 matmul of those rows."""
  rows, k, n = 98304, 16384, 256
  gen = torch.Generator(device="cuda")
  gen.manual_seed(5)
  x = torch.empty((1, rows, k), dtype=torch.bfloat16, device="cuda")
  for i in range(0, rows, 8192):     # in pieces: no float32 copy of 6 GB
    x[0, i:i + 8192] = torch.randn((8192, k), generator=gen,
                                   device="cuda").to(torch.bfloat16)
  w = (torch.randn((k, n), generator=gen, device="cuda") / k ** 0.5).to(
      torch.bfloat16)
  wp = hip.pack_weights(w.reshape(1, k, n), torch.bfloat16)
  y = hip.dense(x, wp, None)
  for sl in (slice(0, 64), slice(rows - 64, rows), slice(65500, 65600)):
    want = x[0, sl].float() @ w.float()
    np.testing.assert_allclose(H.to_np(y[0, sl]), H.to_np(want), rtol=2e-2,
                               atol=2e-2)


@pytest.mark.parametrize("case", [("float32", True), ("bfloat16", False)],
                         ids=["float32-causal", "bfloat16"])
def test_experts_self_attention_layer(case):
  """ExpertsSelfAttention in a layer stack: queries and keys (= values) come
  out of a switch-gated experts layer with two output kernels, the scaled
  queries attend, "o" projects back; against the oracle."""
  act_dtype, autoregressive = case
  b, l, m, e, hdim, heads, d, group = 2, 64, 64, 4, 96, 4, 16, 32
  rng = np.random.default_rng(31)
  n = lambda *shape: H.normal_weights(rng, shape, shape[-2])
  w = dict(w_gate=n(m, e), wi=n(e, m, hdim), q_wo=n(e, hdim, heads * d),
           k_wo=n(e, hdim, heads * d), o=n(heads * d, m))
  scale = (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  final = (1 + 0.1 * rng.standard_normal(m)).astype(np.float32)
  # tokens whose normalised form keeps every router decision clear
  for _ in range(100):
    x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), act_dtype)
    xn = B.rms_norm(x, scale, act_dtype)
    lg = np.sort(O.router_logits(xn.reshape(-1, group, m),
                                 O.cast_act(w["w_gate"], act_dtype)), axis=-1)
    if (lg[..., -1] - lg[..., -2]).min() > (2e-2 if act_dtype == "bfloat16"
                                           else 1e-3):
      break
  hp_kw = dict(moe_gating="switch", moe_num_experts=e, moe_hidden_size=hdim,
               moe_group_size=group, moe_capacity_factor_eval=1.25,
               moe_switch_policy_train="argmax", moe_switch_policy_eval="argmax",
               moe_use_experts_attention=True, moe_min_expert_capacity=4,
               moe_loss_coef=1e-2)
  ohp = O.default_hparams(**hp_kw)
  dt = H.ACT_TORCH[act_dtype]
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(transformer_layers.ExpertsSelfAttention,
        dict(num_heads=heads, key_value_size=d, shared_kv=True, num_experts=e,
             hidden_size=hdim, group_size=group, capacity_factor_eval=1.25,
             switch_policy_train="argmax", switch_policy_eval="argmax"))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=autoregressive)
  y, losses = model.call_layers(
      xt, mtf.VariableDType(torch.float32, torch.float32, dt), mode="eval")
  p = "decoder/layer_000/ExpertsSelfAttention/"
  init = {"decoder/rms_norm/scale": final,
          "decoder/layer_000/rms_norm/scale": scale,
          p + "switch_gating/kernel": w["w_gate"], p + "wi/kernel": w["wi"],
          p + "q_wo/kernel": w["q_wo"], p + "k_wo/kernel": w["k_wo"],
          p + "o": w["o"]}
  assert sorted(init) == sorted(v.name for v in graph.all_variables)
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = H.to_np(lowering.export_to_tf_tensor(y))
  assert len(losses) == 1
  got_loss = float(H.to_np(lowering.export_to_tf_tensor(losses[0])))
  # the oracle's stack: x + layer(rms_norm(x)), then the final rms_norm
  att, want_loss = B.experts_self_attention(
      B.rms_norm(x, scale, act_dtype), w["w_gate"], w["wi"], w["q_wo"],
      w["k_wo"], w["o"], ohp, heads, autoregressive, act_dtype)
  want = B.rms_norm(O.cast_act(x + att, act_dtype), final, act_dtype)
  tol = dict(rtol=2e-4, atol=2e-4) if act_dtype == "float32" else dict(
      rtol=5e-2, atol=5e-2)
  np.testing.assert_allclose(got, want, **tol)
  np.testing.assert_allclose(got_loss, want_loss,
                             rtol=1e-4 if act_dtype == "float32" else 2e-2)
  with pytest.raises(ValueError, match="shared_kv must be True"):
    g2 = mtf.Graph()
    x2 = mtf.import_tf_tensor(mtf.Mesh(g2, "mesh"), torch.zeros(b, l, m),
                              mtf.Shape(dims))
    st2 = transformer.make_layer_stack(
        [(transformer_layers.ExpertsSelfAttention, dict(num_heads=heads))],
        num_layers=1, block_scope=False)
    transformer.Unitransformer(st2, d_model=m, name="decoder").call_layers(
        x2, mtf.VariableDType(torch.float32), mode="eval")


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_broadcast_dropout_entry(hip, act_dtype):
  """mesh_moe_broadcast_dropout: x [outer, mid, inner] times the noise of a
  uniform draw [outer, inner], against the oracle; then the same multiplier
  passed back in (the backward pass)."""
  dt = H.ACT_TORCH[act_dtype]
  rng = np.random.default_rng(41)
  for outer, mid, inner, keep in ((3, 5, 16, 0.75), (2, 7, 24, 0.9),
                                  (6, 4, 1, 0.5), (1, 1, 40, 0.9),
                                  (2, 3, 5, 0.6), (4, 33, 256, 0.9)):
    x = O.cast_act(rng.standard_normal((outer, mid, inner)).astype(np.float32),
                   act_dtype)
    u = O.cast_act(rng.random((outer, inner)).astype(np.float32), act_dtype)
    noise = O.hidden_dropout_noise(u, keep, act_dtype)
    want = B.broadcast_dropout(x, noise, 1, act_dtype)
    xt = torch.from_numpy(x).to(dt).cuda()
    got, got_noise = hip.broadcast_dropout(
        xt, (outer, mid, inner), uniform=torch.from_numpy(u).to(dt).cuda(),
        keep_prob=keep, want_noise=True)
    np.testing.assert_array_equal(H.to_np(got_noise), noise)
    np.testing.assert_array_equal(H.to_np(got), want)
    assert 0 < (noise == 0).sum() < noise.size or noise.size < 8
    dy = O.cast_act(rng.standard_normal(x.shape).astype(np.float32), act_dtype)
    back, same = hip.broadcast_dropout(torch.from_numpy(dy).to(dt).cuda(),
                                       (outer, mid, inner), noise=got_noise)
    assert same is got_noise
    np.testing.assert_array_equal(
        H.to_np(back), B.broadcast_dropout(dy, noise, 1, act_dtype))
  with pytest.raises(hip.MoeHipError, match="exactly one"):
    hip.broadcast_dropout(xt, (4, 33, 256))
  with pytest.raises(hip.MoeHipError, match="do not cover"):
    hip.broadcast_dropout(xt, (4, 33, 255), noise=got_noise)
  with pytest.raises(hip.MoeHipError, match="keep_prob"):
    hip.broadcast_dropout(xt, (4, 33, 256),
                          uniform=torch.zeros((4, 256), dtype=dt,
                                              device="cuda"), keep_prob=0.0)


def test_dropout_operation_and_gradient():
  """mtf.dropout through the graph: noise shared along `length`, the saved
  multiplier, the gradient, and the cases that return x or raise."""
  b, l, m = 2, 6, 16
  rng = np.random.default_rng(42)
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  dy = rng.standard_normal((b, l, m)).astype(np.float32)
  u = rng.random((b, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy), mtf.Shape(dims))
  assert mtf.dropout(xt, False, rate=0.5) is xt
  assert mtf.dropout(xt, True, keep_prob=1.0) is xt
  with pytest.raises(ValueError, match="exactly one"):
    mtf.dropout(xt, True)
  with pytest.raises(ValueError, match="exactly one"):
    mtf.dropout(xt, True, keep_prob=0.5, rate=0.5)
  with pytest.raises(ValueError, match="not a subset"):
    mtf.dropout(xt, True, rate=0.5,
                noise_shape=mtf.Shape([mtf.Dimension("other", 3)]))
  y = mtf.dropout(xt, True, rate=0.25,
                  noise_shape=mtf.Shape([dims[0], dims[2]]))
  op = y.operation
  assert op.sizes == (b, l, m)
  op.uniform = torch.from_numpy(u).cuda()
  y_all = mtf.dropout(xt, True, keep_prob=0.5)            # noise of x's shape
  assert y_all.operation.sizes == (1, 1, b * l * m)
  y_last = mtf.dropout(xt, True, keep_prob=0.5,
                       noise_shape=mtf.Shape(dims[:2]))   # shared by channels
  assert y_last.operation.sizes == (b * l, m, 1)
  (dx,) = mtf.gradients([y], [xt], [dyt])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()})
  noise = O.hidden_dropout_noise(u, 0.75, "float32")
  np.testing.assert_array_equal(H.to_np(op.noise), noise)
  np.testing.assert_array_equal(H.to_np(lowering.export_to_tf_tensor(y)),
                                B.broadcast_dropout(x, noise, 1))
  np.testing.assert_array_equal(H.to_np(lowering.export_to_tf_tensor(dx)),
                                B.broadcast_dropout(dy, noise, 1))
  got = H.to_np(lowering.export_to_tf_tensor(y_all))
  n_all = H.to_np(y_all.operation.noise).reshape(x.shape)
  assert set(np.unique(n_all)) == {0.0, 2.0}
  np.testing.assert_array_equal(got, x * n_all)
  got = H.to_np(lowering.export_to_tf_tensor(y_last))
  n_last = H.to_np(y_last.operation.noise).reshape(b, l, 1)
  np.testing.assert_array_equal(got, x * n_last)
  # a 4-d tensor with noise over dimensions 0 and 2 leaves two separate runs out
  graph2 = mtf.Graph()
  mesh2 = mtf.Mesh(graph2, "mesh")
  d4 = dims + [mtf.Dimension("extra", 2)]
  x4 = mtf.import_tf_tensor(mesh2, torch.zeros((b, l, m, 2)), mtf.Shape(d4))
  with pytest.raises(NotImplementedError, match="not consecutive"):
    mtf.dropout(x4, True, rate=0.5, noise_shape=mtf.Shape([d4[0], d4[2]]))


def test_layer_stack_with_dropout():
  """A training-mode stack with every dropout of the block switched on: the
  sublayer dropouts (noise per batch entry and channel), the attention
  weights' (noise per batch entry, head and memory position, applied to the
  values here) and DenseReluDense's hidden one; the oracle gets the multipliers
  the lowering drew."""
  import functools
  b, l, m, e, hdim, heads, d, group = 2, 64, 64, 4, 96, 4, 16, 32
  rng = np.random.default_rng(43)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  layers = [layers[0], layers[3], layers[1]]      # attention, dense, MoE
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  drop = functools.partial(transformer.sublayer_dropout, dropout_rate=0.2)
  stack_cls = functools.partial(
      transformer.LayerStack, sublayers_initial=[drop],
      sublayers_per_layer=[transformer.sublayer_rms_norm,
                           transformer.sublayer_call_layer, drop,
                           transformer.sublayer_residual],
      sublayers_final=[transformer.sublayer_rms_norm, drop])
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention,
        dict(num_heads=heads, key_value_size=d, dropout_rate=0.3)),
       (transformer_layers.DenseReluDense,
        dict(hidden_size=hdim, dropout_rate=0.4)),
       (moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                        second_policy_train="all", second_policy_eval="all",
                        capacity_factor_train=2.0))],
      num_layers=1, block_scope=False, layer_stack_cls=stack_cls)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=True)
  y, losses = model.call_layers(
      xt, mtf.VariableDType(torch.float32), mode="train")
  init = {"decoder/rms_norm/scale": final}
  for i, (layer, cls) in enumerate(zip(layers, ("SelfAttention",
                                                "DenseReluDense", "MoE1D"))):
    p = "decoder/layer_%03d/" % i
    init[p + "rms_norm/scale"] = layer["scale"]
    if cls == "SelfAttention":
      for k in "qkvo":
        init[p + cls + "/" + k] = layer["w" + k]
    elif cls == "MoE1D":
      init[p + cls + "/top_2_gating/kernel"] = layer["w_gate"]
      init[p + cls + "/wi/kernel"] = layer["wi"]
      init[p + cls + "/wo/kernel"] = layer["wo"]
    else:
      init[p + cls + "/wi/kernel"] = layer["wi"]
      init[p + cls + "/wo/kernel"] = layer["wo"]
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = H.to_np(lowering.export_to_tf_tensor(y))
  drops = [op for op in graph.operations
           if isinstance(op, mtf.DropoutOperation)]
  # graph order: initial; attention's, its sublayer's; hidden, its sublayer's;
  # the MoE layer's sublayer's; final
  assert [op.keep_prob for op in drops] == [0.8, 0.7, 0.8, 0.6, 0.8, 0.8, 0.8]
  noises = [H.to_np(op.noise) for op in drops]
  assert noises[1].shape == (b * l * heads, 1)
  layers[0] = dict(layers[0], sublayer_noise=noises[2],
                   weights_noise=noises[1].reshape(b, l, heads).transpose(
                       0, 2, 1))
  layers[1] = dict(layers[1], hidden_noise=noises[3], sublayer_noise=noises[4])
  hp = O.default_hparams(
      moe_num_experts=e, moe_hidden_size=hdim, moe_group_size=group,
      moe_second_policy_eval="all", moe_second_policy_train="all",
      moe_capacity_factor_train=2.0)
  layers[2] = dict(layers[2], sublayer_noise=noises[5], hparams=hp)
  want, want_loss = B.layer_stack(x, layers, final, "float32", True, True,
                                  initial_noise=noises[0],
                                  final_noise=noises[6])
  for noise, keep in zip(noises, (0.8, 0.7, 0.8, 0.6, 0.8, 0.8, 0.8)):
    assert 0.3 < (noise == 0).mean() / (1 - keep) < 2.0
  np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
  got_loss = [float(H.to_np(lowering.export_to_tf_tensor(t))) for t in losses]
  np.testing.assert_allclose(got_loss, want_loss, rtol=1e-4)


@pytest.mark.parametrize("act_dtype", ["float32", "bfloat16"])
def test_block_backward_entries(hip, act_dtype):
  """rms_norm_backward, dense_backward (with and without relu) and
  self_attention_backward (both visibility modes) against the oracle."""
  dt = H.ACT_TORCH[act_dtype]
  tol = dict(rtol=2e-4, atol=2e-4) if act_dtype == "float32" else dict(
      rtol=3e-2, atol=3e-2)
  rng = np.random.default_rng(51)
  dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dt).cuda()
  rnd = lambda *s: O.cast_act(rng.standard_normal(s).astype(np.float32),
                              act_dtype)
  for rows, m in ((37, 48), (1024, 256), (5, 1000), (300, 512), (2100, 1536),
                  (1030, 4096), (3, 2048)):
    x, dy = rnd(rows, m), rnd(rows, m)
    scale = O.cast_act((1 + 0.2 * rng.standard_normal(m)).astype(np.float32),
                       act_dtype)
    dx, ds = hip.rms_norm_backward(dev(x), dev(scale), dev(dy))
    want_dx, want_ds = B.rms_norm_backward(x, scale, dy, act_dtype)
    np.testing.assert_allclose(H.to_np(dx), want_dx, **tol)
    np.testing.assert_allclose(H.to_np(ds), want_ds, rtol=tol["rtol"],
                               atol=tol["atol"] * rows ** 0.5)
  b, l, k, n = 2, 64, 128, 192
  x, dy = rnd(b, l, k), rnd(b, l, n)
  w = O.cast_act(H.normal_weights(rng, (k, n), k), act_dtype)
  for act in (None, "relu"):
    y = B.dense(x, w, act_dtype, act)
    dx, dw = hip.dense_backward(dev(x), dev(w), dev(dy),
                                dev(y) if act else None)
    want_dx, want_dw = B.dense_backward(x, w, dy, act_dtype, act)
    np.testing.assert_allclose(H.to_np(dx), want_dx, **tol)
    np.testing.assert_allclose(H.to_np(dw), want_dw, rtol=tol["rtol"],
                               atol=tol["atol"] * 4)
  for bsz, length, heads, d, causal in ((2, 64, 4, 16, True),
                                        (1, 128, 2, 64, False),
                                        (2, 256, 2, 128, True),
                                        (1, 512, 2, 64, True),
                                        (1, 1024, 1, 64, False)):
    q, kk, v, do = (rnd(bsz, length, heads * d) * np.float32(0.5)
                    for _ in range(4))
    q, kk, v, do = (O.cast_act(t, act_dtype) for t in (q, kk, v, do))
    got = hip.self_attention_backward(dev(q), dev(kk), dev(v), dev(do), heads,
                                      causal)
    want = B.attention_core_backward(q, kk, v, do, heads, causal, act_dtype)
    for g, wnt, name in zip(got, want, "qkv"):
      np.testing.assert_allclose(H.to_np(g), wnt, err_msg="d" + name, **tol)
    w_got = hip.attention_weights(dev(q), dev(kk), heads, causal)
    np.testing.assert_allclose(H.to_np(w_got).sum(-1), 1.0,
                               rtol=1e-5 if act_dtype == "float32" else 2e-2)


@pytest.mark.parametrize("bsz,length,heads,d,causal", [
    (1, 8, 1, 64, True), (2, 72, 2, 64, False), (1, 200, 3, 128, True),
    (1, 328, 2, 128, False), (2, 256, 2, 64, True), (1, 776, 1, 128, True),
    (1, 1280, 2, 64, False)])
def test_fused_attention_backward(hip, bsz, length, heads, d, causal):
  """mesh_moe_self_attention_backward (nothing [L, L] in memory) against the
  oracle and against the composed path, bf16, lengths that are not multiples
  of the kernels' tiles (64 streamed rows, 256 own rows)."""
  rng = np.random.default_rng(length + d)
  dt = torch.bfloat16
  mk = lambda: O.cast_act(
      (rng.standard_normal((bsz, length, heads * d)) * 0.5).astype(np.float32),
      "bfloat16")
  q, kk, v, do = mk(), mk(), mk(), mk()
  dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dt).cuda()
  args = (dev(q), dev(kk), dev(v), dev(do), heads, causal)
  got = hip.self_attention_backward(*args, fused=True)
  want = B.attention_core_backward(q, kk, v, do, heads, causal, "bfloat16")
  composed = hip.self_attention_backward(*args, fused=False)
  for g, wnt, c, name in zip(got, want, composed, "qkv"):
    scale = max(1.0, float(np.abs(wnt).max()))
    np.testing.assert_allclose(H.to_np(g), wnt, rtol=3e-2, atol=3e-2 * scale,
                               err_msg="d" + name)
    # the two device paths differ by a few roundings only
    diff = np.abs(H.to_np(g) - H.to_np(c))
    assert float(diff.mean()) < 4e-3 * scale, (name, float(diff.mean()))
  # the same bits on every run (no atomics)
  again = hip.self_attention_backward(*args, fused=True)
  for g, a in zip(got, again):
    assert torch.equal(g, a)
  # with the forward pass's outputs and softmax denominators handed back, the
  # pass that recomputes them drops out: lse is the same number, delta comes
  # from the rounded outputs
  out, lse = hip.self_attention(*args[:3], heads, causal, return_lse=True)
  assert torch.equal(out, hip.self_attention(*args[:3], heads, causal))
  qf, kf = (t.reshape(bsz, length, heads, d).astype(np.float64) for t in (q, kk))
  logits = np.einsum("blhd,bmhd->bhlm", qf, kf)
  if causal:
    logits = np.where(np.tril(np.ones((length, length), bool)), logits, -np.inf)
  mx = logits.max(-1, keepdims=True)
  want_lse = (mx + np.log(np.exp(logits - mx).sum(-1, keepdims=True)))[..., 0]
  np.testing.assert_allclose(H.to_np(lse).reshape(bsz, heads, length), want_lse,
                             rtol=1e-5, atol=1e-5)
  saved = hip.self_attention_backward(*args, fused=True, out=out, lse=lse)
  for g, sv, wnt, name in zip(got, saved, want, "qkv"):
    scale = max(1.0, float(np.abs(wnt).max()))
    np.testing.assert_allclose(H.to_np(sv), wnt, rtol=3e-2, atol=3e-2 * scale,
                               err_msg="saved d" + name)
    diff = np.abs(H.to_np(g) - H.to_np(sv))
    assert float(diff.mean()) < 2e-3 * scale, (name, float(diff.mean()))
  with pytest.raises(hip.MoeHipError):
    hip.self_attention_backward(*(t.float() if isinstance(t, torch.Tensor)
                                  else t for t in args), fused=True)


@pytest.mark.parametrize("with_ids_and_bias", [False, True])
def test_attention_gradient_graph_keeps_the_denominators(with_ids_and_bias):
  """Through the graph API with shapes the fused kernels take (bf16, d_kv 64):
  once mtf.gradients has been called, the attention operation keeps lse and
  its outputs for the backward pass.  The gradients must be those of the same
  graph lowered with that switched off (the backward pass then recomputes
  them), up to the rounding of the outputs delta is formed from."""
  b, l, m, heads, d = 2, 136, 64, 2, 64
  rng = np.random.default_rng(91)
  dt = torch.bfloat16
  x = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), "bfloat16")
  dy = O.cast_act(rng.standard_normal((b, l, m)).astype(np.float32), "bfloat16")
  ids = _packed_sequence_ids(rng, b, l, 50) if with_ids_and_bias else None
  results = []
  for keep in (True, False):
    graph = mtf.Graph()
    mesh = mtf.Mesh(graph, "mesh")
    dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
            mtf.Dimension("d_model", m)]
    xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
    dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy).to(dt), mtf.Shape(dims))
    idt = None
    if ids is not None:
      idt = mtf.import_tf_tensor(mesh, torch.from_numpy(ids), mtf.Shape(dims[:2]))
    kw = dict(num_heads=heads, key_value_size=d)
    if with_ids_and_bias:
      kw.update(relative_attention_type="bias", relative_attention_num_buckets=8)
    stack = transformer.make_layer_stack(
        [(transformer_layers.SelfAttention, kw)], num_layers=1, block_scope=False)
    model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                       autoregressive=True)
    y, _ = model.call_layers(xt, mtf.VariableDType(torch.float32, torch.float32, dt),
                             mode="eval", sequence_id=idt)
    variables = sorted(graph.trainable_variables, key=lambda v: v.name)
    grads = mtf.gradients([y], [xt] + [v.outputs[0] for v in variables], [dyt])
    att = [op for op in graph.operations
           if type(op).__name__ == "SelfAttentionOperation"]
    assert len(att) == 1 and att[0]._save_for_backward
    att[0]._save_for_backward = keep
    init_rng = np.random.default_rng(92)
    init = {v.name: H.normal_weights(init_rng, tuple(v.shape.to_integer_list),
                                     v.shape.to_integer_list[0])
            if v.shape.ndims == 2 else np.ones(v.shape.to_integer_list, np.float32)
            for v in variables}
    lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
    saved = lowering.operations[att[0]]
    results.append([H.to_np(lowering.export_to_tf_tensor(t)) for t in [y] + grads])
    assert not saved        # used up by the backward pass, or never kept
  names = ["y", "dx"] + [v.name for v in variables]
  for kept, plain, name in zip(results[0], results[1], names):
    assert np.isfinite(kept).all()
    scale = max(1e-3, float(np.abs(plain).max()))
    diff = np.abs(kept - plain)
    assert float(diff.max()) <= 4e-2 * scale, (name, float(diff.max()), scale)
    assert float(diff.mean()) <= 4e-3 * scale, (name, float(diff.mean()), scale)
  np.testing.assert_array_equal(results[0][0], results[1][0])


def test_layer_stack_gradients():
  """mtf.gradients through a stack of attention and DenseReluDense layers
  (RMS norms, residuals, projections): every variable's gradient and the
  input's against the oracle's per-operation backward passes chained by
  hand, float32."""
  b, l, m, hdim, heads, d = 2, 32, 64, 96, 4, 16
  rng = np.random.default_rng(52)
  layers, final = _build_stack(rng, m, 4, hdim, heads, d, 32)
  att, ffn = layers[0], layers[3]
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  dy = rng.standard_normal((b, l, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention,
        dict(num_heads=heads, key_value_size=d)),
       (transformer_layers.DenseReluDense, dict(hidden_size=hdim))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                     autoregressive=True)
  y, _ = model.call_layers(xt, mtf.VariableDType(torch.float32), mode="eval")
  init = {"decoder/rms_norm/scale": final,
          "decoder/layer_000/rms_norm/scale": att["scale"],
          "decoder/layer_001/rms_norm/scale": ffn["scale"],
          "decoder/layer_001/DenseReluDense/wi/kernel": ffn["wi"],
          "decoder/layer_001/DenseReluDense/wo/kernel": ffn["wo"]}
  for kname in "qkvo":
    init["decoder/layer_000/SelfAttention/" + kname] = att["w" + kname]
  variables = {v.name: v for v in graph.all_variables}
  assert sorted(variables) == sorted(init)
  names = sorted(init)
  grads = mtf.gradients([y], [xt] + [variables[n].outputs[0] for n in names],
                        [dyt])
  # DenseReluDense: the output projection's backward applies the ReLU mask to
  # the hidden gradient, the first projection's backward knows and skips it
  dense_grads = [op for op in graph.operations
                 if type(op).__name__ == "DenseGradOperation"]
  assert sum(op._masks_dx for op in dense_grads) == 1
  assert sum(op._dy_is_masked for op in dense_grads) == 1
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = {n: H.to_np(lowering.export_to_tf_tensor(g))
         for n, g in zip(["x"] + names, grads)}
  # the oracle, forward then backward, by hand
  h1 = B.rms_norm(x, att["scale"])
  q, k, v = (B.dense(h1, att["w" + c]) for c in "qkv")
  o = B._attention_core(q, k, v, heads, True, "float32")
  x1 = x + B.dense(o, att["wo"])
  h2 = B.rms_norm(x1, ffn["scale"])
  hid = B.dense(h2, ffn["wi"], activation="relu")
  x2 = x1 + B.dense(hid, ffn["wo"])
  want = {}
  dx2, want["decoder/rms_norm/scale"] = B.rms_norm_backward(x2, final, dy)
  dhid, want["decoder/layer_001/DenseReluDense/wo/kernel"] = B.dense_backward(
      hid, ffn["wo"], dx2)
  dh2, want["decoder/layer_001/DenseReluDense/wi/kernel"] = B.dense_backward(
      h2, ffn["wi"], dhid, activation="relu")
  d1, want["decoder/layer_001/rms_norm/scale"] = B.rms_norm_backward(
      x1, ffn["scale"], dh2)
  dx1 = dx2 + d1
  do, want["decoder/layer_000/SelfAttention/o"] = B.dense_backward(
      o, att["wo"], dx1)
  dq, dk, dv = B.attention_core_backward(q, k, v, do, heads, True)
  dh1 = 0
  for c, g in zip("qkv", (dq, dk, dv)):
    part, want["decoder/layer_000/SelfAttention/" + c] = B.dense_backward(
        h1, att["w" + c], g)
    dh1 = dh1 + part
  d0, want["decoder/layer_000/rms_norm/scale"] = B.rms_norm_backward(
      x, att["scale"], dh1)
  want["x"] = dx1 + d0
  for name in ["x"] + names:
    scale = max(1.0, float(np.abs(want[name]).max()))
    np.testing.assert_allclose(got[name], want[name], rtol=1e-3,
                               atol=1e-3 * scale, err_msg=name)


def test_layer_stack_gradients_through_moe():
  """mtf.gradients of the output and the MoE loss through rms_norm -> MoE1D
  -> residual -> final rms_norm: the block operations' and the MoE layer's
  backward passes chained by the graph, against the oracles chained by hand."""
  b, l, m, e, hdim, group = 2, 64, 64, 4, 96, 32
  rng = np.random.default_rng(53)
  layers, final = _build_stack(rng, m, e, hdim, 4, 16, group)
  mo = layers[1]
  x = rng.standard_normal((b, l, m)).astype(np.float32)
  dy = rng.standard_normal((b, l, m)).astype(np.float32)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
          mtf.Dimension("d_model", m)]
  xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x), mtf.Shape(dims))
  dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                        second_policy_train="all", second_policy_eval="all",
                        capacity_factor_eval=2.0))],
      num_layers=1, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=m, name="decoder")
  y, losses = model.call_layers(xt, mtf.VariableDType(torch.float32),
                                mode="eval")
  p = "decoder/layer_000/"
  init = {"decoder/rms_norm/scale": final, p + "rms_norm/scale": mo["scale"],
          p + "MoE1D/top_2_gating/kernel": mo["w_gate"],
          p + "MoE1D/wi/kernel": mo["wi"], p + "MoE1D/wo/kernel": mo["wo"]}
  variables = {v.name: v for v in graph.all_variables}
  names = sorted(init)
  assert sorted(variables) == names and len(losses) == 1
  grads = mtf.gradients([y, losses[0]],
                        [xt] + [variables[n].outputs[0] for n in names],
                        [dyt, None])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()}, initial_values=init)
  got = {n: H.to_np(lowering.export_to_tf_tensor(g))
         for n, g in zip(["x"] + names, grads)}
  hp = mo["hparams"]
  h = B.rms_norm(x, mo["scale"])
  out, _, aux = O.moe_layer_v1(h, mo["w_gate"], mo["wi"], mo["wo"], hp, False,
                               "float32", dense=False)
  top = -np.sort(-aux["logits"], axis=-1)[..., :3]
  assert ((top[..., :-1] - top[..., 1:]) > 1e-4).all()   # no near-tied routing
  x1 = x + out
  want = {}
  dx1, want["decoder/rms_norm/scale"] = B.rms_norm_backward(x1, final, dy)
  # the loss reaches the graph multiplied by moe_loss_coef inside the layer;
  # its gradient is seeded with 1
  g = O.moe_layer_v1_backward(h, mo["w_gate"], mo["wi"], mo["wo"], hp, False,
                              "float32", dx1, d_loss=1.0)
  want[p + "MoE1D/top_2_gating/kernel"] = g["dw_gate"]
  want[p + "MoE1D/wi/kernel"] = g["dwi"]
  want[p + "MoE1D/wo/kernel"] = g["dwo"]
  d0, want[p + "rms_norm/scale"] = B.rms_norm_backward(x, mo["scale"], g["dx"])
  want["x"] = dx1 + d0
  for name in ["x"] + names:
    scale = max(1.0, float(np.abs(want[name]).max()))
    np.testing.assert_allclose(got[name], want[name], rtol=1e-3,
                               atol=1e-3 * scale, err_msg=name)


def test_layer_stack_gradients_bfloat16_follow_float32():
  """The whole lm_moe block (attention, MoE1D, attention, DenseReluDense) in
  bfloat16: every gradient is finite, has its variable's shape and points the
  way the float32 gradient of the same graph does (cosine > 0.97; routing may
  differ for a few nearly tied tokens)."""
  b, l, m, e, hdim, heads, d, group = 2, 128, 128, 4, 256, 4, 32, 64
  rng = np.random.default_rng(54)
  layers, final = _build_stack(rng, m, e, hdim, heads, d, group)
  x = O.round_bf16(rng.standard_normal((b, l, m)).astype(np.float32))
  dy = O.round_bf16(rng.standard_normal((b, l, m)).astype(np.float32))

  def run(dt):
    graph = mtf.Graph()
    mesh = mtf.Mesh(graph, "mesh")
    dims = [mtf.Dimension("batch", b), mtf.Dimension("length", l),
            mtf.Dimension("d_model", m)]
    xt = mtf.import_tf_tensor(mesh, torch.from_numpy(x).to(dt), mtf.Shape(dims))
    dyt = mtf.import_tf_tensor(mesh, torch.from_numpy(dy).to(dt),
                               mtf.Shape(dims))
    att = (transformer_layers.SelfAttention,
           dict(num_heads=heads, key_value_size=d))
    stack = transformer.make_layer_stack(
        [att,
         (moe.MoE1D, dict(num_experts=e, hidden_size=hdim, group_size=group,
                          second_policy_train="all", second_policy_eval="all",
                          capacity_factor_eval=2.0)),
         att, (transformer_layers.DenseReluDense, dict(hidden_size=hdim))],
        num_layers=1, block_scope=False)
    model = transformer.Unitransformer(stack, d_model=m, name="decoder",
                                       autoregressive=True)
    y, losses = model.call_layers(
        xt, mtf.VariableDType(torch.float32, torch.float32, dt), mode="eval")
    init = {"decoder/rms_norm/scale": final}
    for i, layer in enumerate(layers):
      p = "decoder/layer_%03d/" % i
      init[p + "rms_norm/scale"] = layer["scale"]
      if layer["kind"] == "attention":
        for kname in "qkvo":
          init[p + "SelfAttention/" + kname] = layer["w" + kname]
      elif layer["kind"] == "moe":
        init[p + "MoE1D/top_2_gating/kernel"] = layer["w_gate"]
        init[p + "MoE1D/wi/kernel"] = layer["wi"]
        init[p + "MoE1D/wo/kernel"] = layer["wo"]
      else:
        init[p + "DenseReluDense/wi/kernel"] = layer["wi"]
        init[p + "DenseReluDense/wo/kernel"] = layer["wo"]
    variables = {v.name: v for v in graph.all_variables}
    names = sorted(init)
    grads = mtf.gradients([y] + list(losses),
                          [xt] + [variables[n].outputs[0] for n in names],
                          [dyt] + [None] * len(losses))
    lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()},
                            initial_values=init)
    out = {}
    for n, g in zip(["x"] + names, grads):
      shape = x.shape if n == "x" else np.shape(init[n])
      value = H.to_np(lowering.export_to_tf_tensor(g))
      assert value.shape == tuple(shape), n
      out[n] = value
    return out

  ref = run(torch.float32)
  got = run(torch.bfloat16)
  for name, want in ref.items():
    g = got[name].astype(np.float64).ravel()
    w = want.astype(np.float64).ravel()
    assert np.isfinite(g).all(), name
    cos = float(g @ w / (np.linalg.norm(g) * np.linalg.norm(w) + 1e-30))
    assert cos > 0.97, (name, cos)
