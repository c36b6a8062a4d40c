"""HipMeshImpl as a MeshImpl plugin: an Operation written against the
reference's interface (mesh_tensorflow/ops.py:1019-1340,
placement_mesh_impl.py:159-355) lowers through every method its lower() may
call.  A mesh of one processor can still have an axis (shape "all:1"), which is
what the axis-taking methods are exercised on."""

import pytest
import torch

import mesh_amd as mtf

pytestmark = pytest.mark.gpu


class _ProbeOperation(mtf.Operation):
  """lower() walks the plugin interface and records what each call returned."""

  def __init__(self, x, new_shape):
    super(_ProbeOperation, self).__init__([x], name="probe")
    self._new_shape = new_shape
    self._outputs = [mtf.Tensor(self, new_shape, x.dtype)]
    self.seen = {}

  def lower(self, lowering):
    impl = lowering.mesh_impl(self)
    x = lowering.tensors[self.inputs[0]]
    seen = self.seen
    seen["delay"] = impl.slicewise_delay_allreduce(lambda t: t * 2, x)
    seen["print"] = impl.Print(x, [x], "message")
    seen["pnum"] = impl.laid_out_pnum()
    seen["pcoord"] = impl.laid_out_pcoord(0)
    seen["slice_num"] = impl.laid_out_slice_num(self.inputs[0].shape)
    seen["allsplit"] = impl.allsplit(x, 0, 0)
    seen["allsplit_which"] = impl.allsplit(x, 0, 1, which=impl.laid_out_pnum())
    seen["allreduce"] = impl.allreduce(x, [0], "SUM")
    seen["allconcat"] = impl.allconcat(x, 0, 0)
    seen["alltoall"] = impl.alltoall(x, 0, 0, 1)
    seen["receive"] = impl.receive(x, 0, [0])
    seen["shift_wrap"] = impl.shift_by_n_processors(x, 0, 1, True)
    seen["shift_pad"] = impl.shift_by_n_processors(x, 0, 1, False)
    seen["einsum"] = impl.slicewise(
        lambda t: impl.einsum("ab,cb->ac", t, t), x)
    out = impl.broadcast_impl(x, self.inputs[0].shape, self._new_shape)
    lowering.set_tensor_lowering(self.outputs[0], out)


def _slice(laid_out):
  return laid_out.to_laid_out_tensor().tensor_list[0]


def test_operation_lowers_through_every_plugin_method():
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  rows, cols = mtf.Dimension("rows", 6), mtf.Dimension("cols", 4)
  value = torch.arange(24, dtype=torch.float32).reshape(6, 4)
  x = mtf.import_tf_tensor(mesh, value, mtf.Shape([rows, cols]))
  new_shape = mtf.Shape([cols, mtf.Dimension("extra", 3), rows])
  op = _ProbeOperation(x, new_shape)
  impl = mtf.HipMeshImpl(shape="all:1", layout="rows:all")
  assert impl.size == 1 and impl.ndims == 1
  assert impl.slice_shape(x.shape) == [6, 4]
  lowering = mtf.Lowering(graph, {mesh: impl})
  v = value.cuda()
  seen = {k: _slice(t) for k, t in op.seen.items()}
  assert torch.equal(seen["delay"], v * 2)
  for name in ("print", "allsplit", "allsplit_which", "allreduce", "allconcat",
               "alltoall", "receive", "shift_wrap"):
    assert torch.equal(seen[name], v), name
  assert torch.equal(seen["shift_pad"], torch.zeros_like(v))
  for name in ("pnum", "pcoord", "slice_num"):
    assert seen[name].dim() == 0 and not seen[name].dtype.is_floating_point
    assert int(seen[name]) == 0, name
  assert torch.equal(seen["einsum"], v @ v.t())
  out = lowering.export_to_tf_tensor(op.outputs[0])
  assert tuple(out.shape) == (4, 3, 6)
  assert torch.equal(out, v.t().reshape(4, 1, 6).expand(4, 3, 6))


def test_generic_slicewise_operation_with_gradient():
  """mtf.slicewise with a grad_function, the hook a fused op attaches to
  (mesh_tensorflow/ops.py:1651-1763), on the empty mesh shape."""
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  dims = [mtf.Dimension("rows", 5), mtf.Dimension("cols", 3)]
  value = torch.linspace(-1, 1, 15).reshape(5, 3)
  x = mtf.import_tf_tensor(mesh, value, mtf.Shape(dims))

  def grad(op, dy):
    return [mtf.slicewise(lambda t, d: 2 * t * d, [op.inputs[0], dy])]

  y = mtf.slicewise(lambda t: t * t, [x], grad_function=grad)
  (dx,) = mtf.gradients([y], [x])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()})
  assert torch.equal(lowering.export_to_tf_tensor(y), value.cuda() ** 2)
  assert torch.equal(lowering.export_to_tf_tensor(dx), 2 * value.cuda())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_multiply_differentiates_both_operands(dtype):
  """mtf.multiply with broadcasting (mesh_tensorflow/ops.py:5135-5153,
  gradient :2044-2084): d(big) = dy * small and d(small) = sum over the
  broadcast dims of dy * big, against float64; a small operand nothing asks a
  gradient for (a mask) gets no reduction op."""
  graph = mtf.Graph()
  mesh = mtf.Mesh(graph, "mesh")
  b, l, m = mtf.Dimension("batch", 3), mtf.Dimension("length", 5), mtf.Dimension("d", 8)
  gen = torch.Generator().manual_seed(4)
  big_v = torch.randn((3, 5, 8), generator=gen).to(dtype)
  small_v = torch.randn((3, 8), generator=gen).to(dtype)
  dy_v = torch.randn((3, 5, 8), generator=gen).to(dtype)
  big = mtf.import_tf_tensor(mesh, big_v, mtf.Shape([b, l, m]))
  small = mtf.import_tf_tensor(mesh, small_v, mtf.Shape([b, m]))
  dy = mtf.import_tf_tensor(mesh, dy_v, mtf.Shape([b, l, m]))
  y = mtf.multiply(big, small)
  d_big, d_small = mtf.gradients([y], [big, small], grad_ys=[dy])
  before = len(graph.operations)
  (only_big,) = mtf.gradients([y], [big], grad_ys=[dy])
  assert not any("mul_grad_small" in op.name
                 for op in graph.operations[before:])
  lowering = mtf.Lowering(graph, {mesh: mtf.HipMeshImpl()})
  want_big = dy_v.double() * small_v.double()[:, None, :]
  want_small = (dy_v.double() * big_v.double()).sum(dim=1)
  tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(
      rtol=2e-2, atol=1e-2)
  for got, want in ((d_big, want_big), (d_small, want_small),
                    (only_big, want_big)):
    out = lowering.export_to_tf_tensor(got)
    assert out.dtype == dtype and tuple(out.shape) == tuple(want.shape)
    torch.testing.assert_close(out.double().cpu(), want, **tol)
