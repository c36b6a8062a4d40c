"""Host-side contract of the mtf-shaped API (no GPU needed): signatures,
defaults, dimension and variable names, error types, and that the C-ABI library
loads and exports every symbol the header declares."""

import ctypes
import inspect
import os
import re

import numpy as np

import pytest
import torch

import mesh_amd as mtf
from mesh_amd import moe_hip
from mesh_amd.transformer import moe

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def hparams(**kw):
  hp = dict(
      moe_gating="top_2", moe_num_experts=8, moe_loss_coef=1e-2,
      moe_hidden_size=64, moe_group_size=32, moe_min_expert_capacity=4,
      moe_capacity_factor_train=1.25, moe_capacity_factor_eval=2.0,
      moe_capacity_factor_second_level=1.0, moe_use_second_place_loss=False,
      moe_second_policy_train="all", moe_second_policy_eval="all",
      moe_second_threshold_train=0.2, moe_second_threshold_eval=0.2,
      moe_dropout_rate=0.0, moe_use_experts_attention=False)
  hp.update(kw)
  return moe.HParams(**hp)


def graph_input(shape=(2, 64, 16), names=("batch", "length", "d_model"),
                dtype=torch.float32):
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension(n, s) for n, s in zip(names, shape)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(shape, dtype=dtype), mtf.Shape(dims))
  return graph, mesh, x, dims


def param_list(fn):
  return [(p.name, p.default) for p in inspect.signature(fn).parameters.values()]


def test_layer_signatures_match_reference():
  """transformer/moe.py:191-194 and :528-530."""
  E = inspect.Parameter.empty
  assert param_list(moe.transformer_moe_layer_v1) == [
      ("inputs", E), ("output_dim", E), ("hparams", E), ("train", E),
      ("variable_dtype", E), ("layout", None), ("mesh_shape", None),
      ("nonpadding", None), ("activation", mtf.relu),
      ("num_microbatches", None)]
  assert param_list(moe.transformer_moe_layer_v2) == [
      ("inputs", E), ("output_dim", E), ("hparams", E), ("train", E),
      ("variable_dtype", E), ("layout", None), ("mesh_shape", None),
      ("nonpadding", None), ("num_microbatches", None)]
  assert param_list(moe._split_into_groups) == [
      ("n", E), ("max_group_size", E), ("mesh_dim_size", E)]


def test_moe1d_moe2d_constructor_defaults():
  """transformer/moe.py:40-64 and :134-147."""
  assert param_list(moe.MoE1D.__init__)[1:] == [
      ("num_experts", 16), ("loss_coef", 1e-2), ("hidden_size", 4096),
      ("group_size", 1024), ("capacity_factor_train", 1.25),
      ("capacity_factor_eval", 2.0), ("use_second_place_loss", False),
      ("second_policy_train", "random"), ("second_policy_eval", "random"),
      ("second_threshold_train", 0.2), ("second_threshold_eval", 0.2),
      ("dropout_rate", 0.0), ("activation", "relu"), ("moe_gating", "top_2"),
      ("min_expert_capacity", 4), ("switch_policy_train", "input_jitter"),
      ("switch_policy_eval", "input_jitter"), ("switch_dropout", 0.1),
      ("switch_temperature", 1.0), ("switch_jitter", 1e-2), ("ntlb_top_k", 4),
      ("output_dim", None), ("use_experts_attention", False), ("z_loss", None)]
  assert param_list(moe.MoE2D.__init__)[1:] == [
      ("expert_x", 8), ("expert_y", 8), ("loss_coef", 1e-2),
      ("hidden_size", 4096), ("group_size", 1024),
      ("capacity_factor_train", 1.25), ("capacity_factor_eval", 2.0),
      ("capacity_factor_second_level", 1.0), ("use_second_place_loss", False),
      ("second_policy_train", "random"), ("second_policy_eval", "random"),
      ("second_threshold_train", 0.2), ("second_threshold_eval", 0.2)]
  hp = moe.MoE1D(num_experts=4)._hparams
  assert hp.moe_num_experts == 4 and hp.moe_gating == "top_2"
  assert moe.MoE2D()._hparams.moe_num_experts == [8, 8]


def test_default_hparams():
  hp = moe.HParams()
  moe.set_default_moe_hparams(hp)
  assert (hp.moe_num_experts, hp.moe_hidden_size, hp.moe_group_size) == (16, 4096, 1024)
  assert hp.moe_capacity_factor_train == 1.25 and hp.moe_capacity_factor_eval == 2.0
  assert hp.moe_second_policy_train == "random" and hp.moe_gating == "top_2"


def test_split_into_groups():
  assert moe._split_into_groups(65536, 2048, 1) == (32, 2048)
  assert moe._split_into_groups(5120, 1024, 1) == (5, 1024)
  # the search starts at n // max_group_size groups, so (as in the reference)
  # a group can exceed max_group_size when that count already divides n
  assert moe._split_into_groups(150, 64, 1) == (2, 75)
  assert moe._split_into_groups(150, 49, 1) == (3, 50)
  assert moe._split_into_groups(96, 32, 4) == (4, 24)
  with pytest.raises(ValueError):
    moe._split_into_groups(10, 4, 3)


def test_v1_switch_graph_names():
  """The switch router's variable lives under "switch_gating" (the `name`
  default of _switch_gating, transformer/moe.py:1179)."""
  graph, _, x, dims = graph_input()
  hp = hparams(moe_gating="switch", moe_switch_policy_train="argmax",
               moe_switch_policy_eval="argmax", moe_z_loss=None)
  with mtf.variable_scope("layer_0"):
    y, loss = moe.transformer_moe_layer_v1(
        x, dims[-1], hp, True, mtf.VariableDType(torch.float32))
  assert y.shape == mtf.Shape(dims) and loss.shape == mtf.Shape([])
  names = sorted(v.name for v in graph.all_variables)
  assert names == ["layer_0/switch_gating/kernel", "layer_0/wi/kernel",
                   "layer_0/wo/kernel"]


def test_v1_gated_activation_graph_names():
  """A list of activations makes one "wi_<i>" dense layer per factor
  (mtf.layers.dense_product, layers.py:293); a list of one keeps "wi"."""
  graph, _, x, dims = graph_input()
  with mtf.variable_scope("layer_0"):
    y, _ = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(), True, mtf.VariableDType(torch.float32),
        activation=["gelu", "linear"])
  assert y.shape == mtf.Shape(dims)
  names = sorted(v.name for v in graph.all_variables)
  assert names == ["layer_0/top_2_gating/kernel", "layer_0/wi_0/kernel",
                   "layer_0/wi_1/kernel", "layer_0/wo/kernel"]
  op = y.operation.inputs[0].operation
  assert [op._activation] + op._more_activations == ["gelu", "linear"]
  grads = mtf.gradients([y], [x] + [v.outputs[0] for v in graph.all_variables])
  assert all(g is not None for g in grads)      # every wi_<i> gets a gradient
  graph2, _, x2, dims2 = graph_input()
  with mtf.variable_scope("layer_0"):
    moe.transformer_moe_layer_v1(
        x2, dims2[-1], hparams(), True, mtf.VariableDType(torch.float32),
        activation=[mtf.relu])
  assert sorted(v.name for v in graph2.all_variables) == [
      "layer_0/top_2_gating/kernel", "layer_0/wi/kernel", "layer_0/wo/kernel"]


def test_v1_ntlb_graph_names():
  """The ntlb router's variable lives under "ntlb_gating" (the `name` default
  of _ntlb_gating, transformer/moe.py:812)."""
  graph, _, x, dims = graph_input()
  hp = hparams(moe_gating="ntlb", moe_switch_policy_train="argmax",
               moe_switch_policy_eval="argmax", moe_ntlb_top_k=3)
  with mtf.variable_scope("layer_0"):
    y, loss = moe.transformer_moe_layer_v1(
        x, dims[-1], hp, True, mtf.VariableDType(torch.float32))
  assert y.shape == mtf.Shape(dims) and loss.shape == mtf.Shape([])
  names = sorted(v.name for v in graph.all_variables)
  assert names == ["layer_0/ntlb_gating/kernel", "layer_0/wi/kernel",
                   "layer_0/wo/kernel"]
  op = [o for o in graph.operations if isinstance(o, moe.MoEV1Operation)][0]
  assert op._gating.top_k == 3


def test_v1_graph_names_and_shapes():
  graph, _, x, dims = graph_input()
  with mtf.variable_scope("layer_0"):
    y, loss = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(), True, mtf.VariableDType(torch.float32))
  assert y.shape == mtf.Shape(dims) and loss.shape == mtf.Shape([])
  got = {v.name: v.shape.to_string for v in graph.all_variables}
  assert got == {
      "layer_0/top_2_gating/kernel": "Shape[d_model=16, expert_unsplit=8]",
      "layer_0/wi/kernel": "Shape[experts=8, d_model=16, expert_hidden=64]",
      "layer_0/wo/kernel": "Shape[experts=8, expert_hidden=64, d_model=16]"}
  op = [o for o in graph.operations if isinstance(o, moe.MoEV1Operation)][0]
  assert op.inputs[0].shape.dimension_names == [
      "outer_batch", "batch", "group", "d_model"]
  assert op.inputs[0].shape.to_integer_list == [1, 4, 32, 16]
  assert op._capacity == 5          # max(min(32, int(32 * 1.25 / 8)), 4)


def test_v2_graph_names_and_shapes():
  graph, _, x, dims = graph_input()
  with mtf.variable_scope("moe2d"):
    y, _ = moe.transformer_moe_layer_v2(
        x, dims[-1], hparams(moe_num_experts=[4, 2]), True,
        mtf.VariableDType(torch.float32))
  assert y.shape == mtf.Shape(dims)
  got = {v.name: v.shape.to_string for v in graph.all_variables}
  assert got == {
      "moe2d/outer_gating/kernel": "Shape[d_model=16, expert_x_unsplit=4]",
      "moe2d/inner_gating/kernel":
          "Shape[expert_x=4, d_model=16, expert_y_unsplit=2]",
      "moe2d/wi/kernel":
          "Shape[expert_y=2, expert_x=4, d_model=16, expert_hidden=64]",
      "moe2d/wo/kernel":
          "Shape[expert_y=2, expert_x=4, expert_hidden=64, d_model=16]"}
  op = [o for o in graph.operations if isinstance(o, moe.MoEV2Operation)][0]
  assert op.inputs[0].shape.dimension_names == [
      "outer_batch", "batch", "group_size_x", "d_model"]
  # x=4, y=2, c=max(min(32, int(32*1.25/4)), 4)=10, 4*10=40 slots -> h0=2,t=20 ...
  assert op._dims[:3] == (4, 2, 10)
  assert op._dims[3] * op._dims[4] == 4 * 10


def test_error_behaviour():
  _, _, x, dims = graph_input()
  vdt = mtf.VariableDType(torch.float32)
  with pytest.raises(ValueError, match="unknown hparams.moe_gating"):
    moe.transformer_moe_layer_v1(x, dims[-1], hparams(moe_gating="top_3"), True, vdt)
  with pytest.raises(ValueError, match="unknown hparams.moe_gating"):
    moe.transformer_moe_layer_v2(
        x, dims[-1], hparams(moe_gating="switch", moe_num_experts=[2, 2]), True, vdt)
  with pytest.raises(ValueError, match="Unknown policy"):
    moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(moe_second_policy_train="sometimes"), True, vdt)
  # ntlb reads the switch policy first, as the reference does (moe.py:816-819)
  with pytest.raises(AttributeError, match="moe_switch_policy_train"):
    moe.transformer_moe_layer_v1(x, dims[-1], hparams(moe_gating="ntlb"), True, vdt)
  # the jitter reads its own hyperparameter, as the reference does
  nt = dict(moe_gating="ntlb", moe_switch_policy_train="input_jitter",
            moe_switch_policy_eval="argmax", moe_ntlb_top_k=2)
  with pytest.raises(AttributeError, match="moe_switch_jitter"):
    moe.transformer_moe_layer_v1(x, dims[-1], hparams(**nt), True, vdt)
  # switch gating reads its own hyperparameters, as the reference does
  with pytest.raises(AttributeError, match="moe_switch_policy_train"):
    moe.transformer_moe_layer_v1(x, dims[-1], hparams(moe_gating="switch"), True, vdt)
  sw = dict(moe_gating="switch", moe_switch_policy_train="argmax",
            moe_switch_policy_eval="sample", moe_z_loss=None)
  # sampling reads its temperature, as the reference does (moe.py:1214-1215)
  with pytest.raises(AttributeError, match="moe_switch_temperature"):
    moe.transformer_moe_layer_v1(x, dims[-1], hparams(**sw), False, vdt)
  with pytest.raises(ValueError, match="Unknown Switch gating policy"):
    moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(**dict(sw, moe_switch_policy_train="best")), True, vdt)
  with pytest.raises(ValueError, match="moe_z_loss needs"):
    moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(**dict(sw, moe_z_loss=1e-3)), True, vdt)
  # dropout on the hidden tensor while training builds (moe.py:477-479)
  with mtf.variable_scope("dropout_train"):
    out, _ = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(moe_dropout_rate=0.1), True, vdt)
  assert out.operation.inputs[0].operation._hidden_keep_prob == 0.9
  with mtf.variable_scope("dropout_eval"):
    out, _ = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(moe_dropout_rate=0.1), False, vdt)
  assert out.operation.inputs[0].operation._hidden_keep_prob is None
  with pytest.raises(ValueError, match="not a multiple of mesh_dim_size"):
    moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(), True, vdt, layout="batch:rows", mesh_shape="rows:3")

  class Model(object):
    ensemble_dim = mtf.Dimension("ensemble", 2)

  class Context(object):
    model = Model()
  with pytest.raises(NotImplementedError, match="ensembles"):
    moe.MoE1D().call(Context(), x)
  with pytest.raises(NotImplementedError, match="ensembles"):
    moe.MoE2D().call(Context(), x)


def test_moe1d_call_adds_length_dim_and_loss():
  graph, _, x, dims = graph_input(shape=(6, 16), names=("batch", "d_model"))

  class Model(object):
    ensemble_dim = None
    model_dim = dims[-1]
    layout = None
    mesh_shape = None

  class Context(object):
    model = Model()
    length_dim = mtf.Dimension("length", 64)
    train = True
    variable_dtype = mtf.VariableDType(torch.float32)
    nonpadding = None
    num_microbatches = None
    losses = []
  layer = moe.MoE1D(num_experts=2, hidden_size=8, group_size=4,
                    second_policy_train="all")
  y = layer.call(Context(), x)
  assert y.shape == x.shape and len(Context.losses) == 1
  op = [o for o in graph.operations if isinstance(o, moe.MoEV1Operation)][0]
  assert op.inputs[0].shape.to_integer_list == [1, 1, 6, 16]


def test_shape_and_layout_helpers():
  s = mtf.convert_to_shape("rows:2,cols:4")
  assert s.size == 8 and s.dimension_names == ["rows", "cols"]
  assert mtf.tensor_dim_to_mesh_dim_size(
      "batch:rows", "rows:2,cols:4", mtf.Dimension("batch", 8)) == 2
  assert mtf.tensor_dim_to_mesh_dim_size(None, None, mtf.Dimension("batch", 8)) == 1
  with pytest.raises(ValueError):
    mtf.Shape([mtf.Dimension("a", 1), mtf.Dimension("a", 2)])
  impl = mtf.MeshImpl("rows:2", "batch:rows")
  assert impl.slice_shape(mtf.Shape([("batch", 8), ("d", 3)])) == [4, 3]
  with pytest.raises(ValueError):
    impl.slice_shape(mtf.Shape([("batch", 7)]))


def test_mesh_impl_interface():
  """The plugin methods an Operation's lower() may call
  (mesh_tensorflow/ops.py:867-1340) exist on HipMeshImpl."""
  for name in ("slicewise", "slicewise_delay_allreduce", "Print", "einsum",
               "allreduce", "allsplit", "allconcat", "alltoall", "receive",
               "shift_by_n_processors", "laid_out_pnum", "laid_out_pcoord",
               "laid_out_slice_num", "broadcast_impl", "import_tf_tensor",
               "export_to_tf_tensor", "slice_shape", "slice_begin",
               "slice_size", "laid_out_size", "tensor_layout",
               "tensor_dimension_to_mesh_axis", "make_slices",
               "combine_slices", "random"):
    assert callable(getattr(mtf.HipMeshImpl, name)), name
  # what HipMeshImpl must supply itself rather than inherit as a stub
  for name in ("slicewise", "einsum", "allreduce", "allconcat", "alltoall",
               "receive", "laid_out_pnum", "import_tf_tensor",
               "export_to_tf_tensor", "random"):
    assert name in vars(mtf.HipMeshImpl), name
  for name in ("shape", "ndims", "size", "layout_rules", "devices",
               "supports_control_dependencies"):
    assert isinstance(getattr(mtf.HipMeshImpl, name), property), name
  for name in ("tensor_list", "all_slices", "slice_shape"):
    assert isinstance(getattr(mtf.HipMeshImpl.LaidOutTensor, name), property)
  assert hasattr(mtf.HipMeshImpl.LaidOutTensor, "to_laid_out_tensor")
  assert hasattr(mtf.HipMeshImpl.LaidOutTensor, "from_tensor_list")
  for name in ("laid_out_tensor", "copy_master_to_slices",
               "copy_slices_to_master", "assign_to_slices"):
    assert hasattr(mtf.HipMeshImpl.LaidOutVariable, name)


def test_no_cpu_fallback():
  if torch.cuda.is_available():
    pytest.skip("a GPU is visible")
  with pytest.raises(RuntimeError, match="needs a GPU"):
    mtf.HipMeshImpl()
  with pytest.raises(moe_hip.MoeHipError):
    moe_hip.router_logits(torch.zeros(4, 8), torch.zeros(8, 2))
  with pytest.raises(moe_hip.MoeHipError, match="not found"):
    moe_hip.load_library("/nonexistent/libmesh_moe_hip.so")


def test_library_exports_every_declared_symbol():
  header = open(os.path.join(ROOT, "include", "mesh_moe.h")).read()
  declared = set(re.findall(r"\b(mesh_moe_[a-z0-9_]+)\s*\(", header))
  assert declared == set(moe_hip.EXPORTS)
  if not os.path.exists(moe_hip.LIB_PATH):
    from mesh_amd.csrc import build
    build.build_library(verbose=False)
  lib = ctypes.CDLL(moe_hip.LIB_PATH)
  for name in declared:
    assert getattr(lib, name) is not None
  lib.mesh_moe_abi_version.restype = ctypes.c_int
  assert lib.mesh_moe_abi_version() == moe_hip.ABI_VERSION
  lib.mesh_moe_gating_workspace_bytes.restype = ctypes.c_size_t
  assert lib.mesh_moe_gating_workspace_bytes(32, 2048, 64) > 0


def test_product_does_not_import_the_oracle():
  pkg = os.path.join(ROOT, "mesh_amd")
  for dirpath, _, files in os.walk(pkg):
    for f in files:
      if f.endswith((".py", ".hip", ".h", ".cpp")):
        text = open(os.path.join(dirpath, f)).read()
        assert "oracle" not in text, os.path.join(dirpath, f)


def test_experts_attention_graph():
  """moe_use_experts_attention returns [q, k] and creates "q_wo" / "k_wo"
  instead of "wo" (transformer/moe.py:514-522)."""
  graph, _, x, dims = graph_input()
  with mtf.variable_scope("att"):
    outs, loss = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(moe_use_experts_attention=True), True,
        mtf.VariableDType(torch.float32))
  assert isinstance(outs, list) and [o.shape for o in outs] == [mtf.Shape(dims)] * 2
  assert loss.shape == mtf.Shape([])
  assert sorted(v.name for v in graph.all_variables) == [
      "att/k_wo/kernel", "att/q_wo/kernel", "att/top_2_gating/kernel",
      "att/wi/kernel"]


def test_gradients_builds_the_backward_operation():
  """mtf.gradients (mesh_tensorflow/ops.py:5254-5291) over the layer: one
  gradient per requested tensor with that tensor's shape and dtype, None for a
  tensor nothing depends on, and the forward operation told to keep its
  activations.  Graph construction only, no GPU."""
  graph, mesh, x, dims = graph_input()
  with mtf.variable_scope("moe"):
    y, loss = moe.transformer_moe_layer_v1(
        x, dims[-1], hparams(), True, mtf.VariableDType(torch.float32))
  variables = [v.outputs[0] for v in graph.trainable_variables]
  other = mtf.import_tf_tensor(mesh, torch.zeros(3), mtf.Shape([mtf.Dimension("z", 3)]))
  grads = mtf.gradients([y, loss], [x] + variables + [other])
  assert grads[-1] is None
  for t, g in zip([x] + variables, grads[:-1]):
    assert g.shape == t.shape and g.dtype == t.dtype
  fwd = [o for o in graph.operations if isinstance(o, moe.MoEV1Operation)][0]
  assert fwd._save_for_backward
  assert any(isinstance(o, moe.MoEV1GradOperation) for o in graph.operations)
  # the second-place loss has a gradient like the rest of the gating
  g2, _, x2, d2 = graph_input()
  y2, l2 = moe.transformer_moe_layer_v1(
      x2, d2[-1], hparams(moe_use_second_place_loss=True), True,
      mtf.VariableDType(torch.float32))
  assert mtf.gradients([y2, l2], [x2])[0].shape == x2.shape
  g3, _, x3, d3 = graph_input()
  y3, l3 = moe.transformer_moe_layer_v2(
      x3, d3[-1], hparams(moe_num_experts=[2, 2]), True,
      mtf.VariableDType(torch.float32))
  v3 = [v.outputs[0] for v in g3.trainable_variables]
  grads3 = mtf.gradients([y3, l3], [x3] + v3)
  assert [g.shape for g in grads3] == [t.shape for t in [x3] + v3]
  assert any(isinstance(o, moe.MoEV2GradOperation) for o in g3.operations)


# ---- the transformer block around the layer -------------------------------------
def _lm_moe_stack():
  from mesh_amd.transformer import transformer, transformer_layers
  return transformer.make_layer_stack(
      [transformer_layers.SelfAttention,
       (moe.MoE1D, dict(num_experts=4, hidden_size=64, group_size=16,
                        second_policy_train="all", second_policy_eval="all")),
       (transformer_layers.SelfAttention, dict(num_heads=4, key_value_size=8)),
       (transformer_layers.DenseReluDense, dict(hidden_size=64))],
      num_layers=1, block_scope=False)


def test_layer_stack_graph_names_and_shapes():
  """The block of transformer/gin/models/lm_moe.gin:11-16: variable names and
  shapes are the reference's (rms_norm/scale per layer and at the end,
  SelfAttention/{q,k,v,o} with heads and d_kv combined, attention.py:410-414)."""
  from mesh_amd.transformer import transformer
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", 2), mtf.Dimension("length", 16),
          mtf.Dimension("d_model", 32)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(2, 16, 32), mtf.Shape(dims))
  model = transformer.Unitransformer(_lm_moe_stack(), d_model=32,
                                     name="decoder", autoregressive=True)
  y, losses = model.call_layers(x, mtf.VariableDType(torch.float32))
  assert y.shape == x.shape and len(losses) == 1
  got = {v.name: v.shape.to_string for v in graph.all_variables}
  assert got == {
      "decoder/layer_000/rms_norm/scale": "Shape[d_model=32]",
      "decoder/layer_000/SelfAttention/q": "Shape[d_model=32, heads=1024]",
      "decoder/layer_000/SelfAttention/k": "Shape[d_model=32, heads=1024]",
      "decoder/layer_000/SelfAttention/v": "Shape[d_model=32, heads=1024]",
      "decoder/layer_000/SelfAttention/o": "Shape[heads=1024, d_model=32]",
      "decoder/layer_001/rms_norm/scale": "Shape[d_model=32]",
      "decoder/layer_001/MoE1D/top_2_gating/kernel":
          "Shape[d_model=32, expert_unsplit=4]",
      "decoder/layer_001/MoE1D/wi/kernel":
          "Shape[experts=4, d_model=32, expert_hidden=64]",
      "decoder/layer_001/MoE1D/wo/kernel":
          "Shape[experts=4, expert_hidden=64, d_model=32]",
      "decoder/layer_002/rms_norm/scale": "Shape[d_model=32]",
      "decoder/layer_002/SelfAttention/q": "Shape[d_model=32, heads=32]",
      "decoder/layer_002/SelfAttention/k": "Shape[d_model=32, heads=32]",
      "decoder/layer_002/SelfAttention/v": "Shape[d_model=32, heads=32]",
      "decoder/layer_002/SelfAttention/o": "Shape[heads=32, d_model=32]",
      "decoder/layer_003/rms_norm/scale": "Shape[d_model=32]",
      "decoder/layer_003/DenseReluDense/wi/kernel": "Shape[d_model=32, d_ff=64]",
      "decoder/layer_003/DenseReluDense/wo/kernel": "Shape[d_ff=64, d_model=32]",
      "decoder/rms_norm/scale": "Shape[d_model=32]"}


@pytest.mark.parametrize("kind", ["bias", "bias_shared"])
def test_relative_attention_bias_variables(kind):
  """compute_bias (transformer_layers.py:317-352): a variable
  "relative_attention_bias" [heads, buckets] per attention layer, or only in
  the first one with "bias_shared"."""
  from mesh_amd.transformer import transformer, transformer_layers
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", 2), mtf.Dimension("length", 16),
          mtf.Dimension("d_model", 32)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(2, 16, 32), mtf.Shape(dims))
  kw = dict(num_heads=4, key_value_size=8, relative_attention_type=kind,
            relative_attention_num_buckets=16)
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention, kw)], num_layers=2, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=32, name="encoder",
                                     autoregressive=False)
  model.call_layers(x, mtf.VariableDType(torch.float32))
  got = {v.name: v.shape.to_string for v in graph.all_variables
         if "relative" in v.name}
  want = {"encoder/layer_000/SelfAttention/relative_attention_bias":
              "Shape[heads=4, buckets=16]"}
  if kind == "bias":
    want["encoder/layer_001/SelfAttention/relative_attention_bias"] = (
        "Shape[heads=4, buckets=16]")
  assert got == want


def test_shared_kv_variables():
  """SelfAttention(shared_kv=True): one kernel "kv" in place of "k" and "v"
  (attention.py:453-459); one recurrent state per layer in the decoding modes
  (transformer_layers.py:244-258)."""
  from mesh_amd.transformer import transformer, transformer_layers
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", 2), mtf.Dimension("length", 16),
          mtf.Dimension("d_model", 32)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(2, 16, 32), mtf.Shape(dims))
  stack = transformer.make_layer_stack(
      [(transformer_layers.SelfAttention,
        dict(num_heads=4, key_value_size=8, shared_kv=True))],
      num_layers=2, block_scope=False)
  model = transformer.Unitransformer(stack, d_model=32, name="decoder",
                                     autoregressive=True)
  states = []
  model.call_layers(x, mtf.VariableDType(torch.float32), mode="first_part",
                    new_states=states)
  assert len(states) == 2
  names = sorted(v.name for v in graph.all_variables
                 if "layer_000/SelfAttention" in v.name)
  assert names == ["decoder/layer_000/SelfAttention/" + n
                   for n in ("kv", "o", "q")]


def test_relative_position_bucket_matches_the_oracle():
  """The host-side bucket table of the product against the oracle's
  restatement of _relative_position_bucket (transformer_layers.py:1000-1042),
  which the CPU tests pin by hand."""
  from mesh_amd.transformer import attention
  from oracle import block_oracle
  rp = np.arange(-3000, 3000)
  for bidirectional in (True, False):
    for nb in (8, 32, 64):
      np.testing.assert_array_equal(
          attention.relative_position_bucket(rp, bidirectional, nb),
          block_oracle.relative_position_bucket(rp, bidirectional, nb))


def test_layer_stack_names_with_block_scope_and_legacy_mode():
  from mesh_amd.transformer import transformer, transformer_layers
  stack = transformer.make_layer_stack(
      [transformer_layers.SelfAttention,
       (transformer_layers.DenseReluDense, "feedforward", {"hidden_size": 8})],
      num_layers=2)
  assert [l.name for l in stack.layers] == [
      "block_000/layer_000", "block_000/feedforward",
      "block_001/layer_000", "block_001/feedforward"]
  legacy = transformer.LayerStack(stack.layers, dropout_rate=0.0,
                                  norm_epsilon=1e-6)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", 1), mtf.Dimension("length", 8),
          mtf.Dimension("d_model", 16)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(1, 8, 16), mtf.Shape(dims))
  model = transformer.Unitransformer(legacy, d_model=16, name="encoder")
  model.call_layers(x, mtf.VariableDType(torch.float32))
  names = [v.name for v in graph.all_variables]
  assert "encoder/block_000/layer_000/layer_norm/scale" in names
  assert "encoder/final_layer_norm/scale" in names
  with pytest.raises(ValueError, match="legacy mode"):
    transformer.LayerStack(stack.layers, dropout_rate=0.1)


def test_block_rejections():
  from mesh_amd.transformer import transformer, transformer_layers
  with pytest.raises(NotImplementedError):
    transformer_layers.SelfAttention(relative_attention_type="contextual")
  with pytest.raises(ValueError, match="unrecognized"):
    transformer_layers.SelfAttention(relative_attention_type="nope")
  with pytest.raises(NotImplementedError):
    transformer_layers.SelfAttention(num_memory_heads=2)
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("batch", 1), mtf.Dimension("length", 8),
          mtf.Dimension("d_model", 16)]
  x = mtf.import_tf_tensor(mesh, torch.zeros(1, 8, 16), mtf.Shape(dims))
  vdt = mtf.VariableDType(torch.float32)
  model = transformer.Unitransformer(None, d_model=16)
  with pytest.raises(ValueError, match="position"):
    transformer.Context(model, mesh, dims[:1], dims[1], vdt, mode="incremental")
  with pytest.raises(ValueError, match="unknown mode"):
    transformer.Context(model, mesh, dims[:1], dims[1], vdt, mode="beam")
  pos = mtf.import_tf_tensor(mesh, torch.zeros(1, dtype=torch.int32),
                             mtf.Shape(dims[:1]))
  ctx = transformer.Context(model, mesh, dims[:1], dims[1], vdt,
                            mode="incremental", position=pos, states=[x, x])
  assert ctx.get_states(2) == [x, x]
  ctx.record_new_states([x])
  assert ctx.get_states(1) == [x]
  with pytest.raises(ValueError, match="states were passed"):
    ctx.get_states(2)
  stack = transformer.make_layer_stack(
      [(transformer_layers.DenseReluDense,
        dict(hidden_size=8, dropout_rate=0.1))], num_layers=1)
  model = transformer.Unitransformer(stack, d_model=16)
  # dropout while training builds mtf.dropout with the noise shared along length
  y, _ = model.call_layers(x, vdt, mode="train")
  drops = [op for op in graph.operations
           if isinstance(op, mtf.DropoutOperation)]
  assert len(drops) == 1 and drops[0].keep_prob == 0.9
  assert drops[0].noise_shape.dimension_names == ["batch", "d_ff"]
  assert drops[0].sizes == (1, 8, 8) and y.shape == x.shape
  ctx = transformer.Context(model, mesh, dims[:1], dims[1], vdt, sequence_id=1)
  assert ctx.nonpadding == 1 and not isinstance(ctx.nonpadding, mtf.Tensor)
  with pytest.raises(ValueError, match="does not end in"):
    model.call_layers(mtf.reshape(x, [dims[0], dims[2], dims[1]]), vdt)


# ---- checkpoints ----------------------------------------------------------------
def test_plan_restore_selection_logic():
  """utils.py:948-972: the filter applies to checkpoint names, the mapping to
  graph names, and only variables that pass should_load are candidates."""
  from mesh_amd import checkpoint
  graph = ["decoder/layer_001/MoE1D/wi/kernel", "decoder/layer_001/MoE1D/wo/kernel",
           "decoder/rms_norm/scale", "decoder/extra/bias"]
  ckpt = ["decoder/layer_001/MoE1D/wi/kernel", "decoder/layer_001/MoE1D/wo/kernel",
          "decoder/rms_norm/scale", "decoder/rms_norm/scale_slot_v", "global_step"]
  r = checkpoint.plan_restore(graph, ckpt)
  assert r.restored == {n: n for n in graph[:3]}
  assert r.in_checkpoint_not_in_graph == ["decoder/rms_norm/scale_slot_v",
                                          "global_step"]
  assert r.in_graph_not_in_checkpoint == ["decoder/extra/bias"]
  r = checkpoint.plan_restore(graph, ckpt, variable_filter=r"MoE1D")
  assert sorted(r.restored) == graph[:2]
  assert r.in_graph_not_in_checkpoint == ["decoder/extra/bias",
                                          "decoder/rms_norm/scale"]
  r = checkpoint.plan_restore(
      ["student/" + n for n in graph], ckpt,
      variable_mapping=lambda n: n[len("student/"):],
      should_load=lambda n: "rms_norm" not in n)
  assert r.restored == {"student/" + n: n for n in graph[:2]}
  assert "decoder/rms_norm/scale" in r.in_checkpoint_not_in_graph
