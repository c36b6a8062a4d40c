"""A small named-dimension graph language with the vocabulary of Mesh TensorFlow.

Only what the Mixture-of-Experts layers need is here: Dimension / Shape /
LayoutRules, Graph / Mesh / Tensor / Operation, variables with master and slice
copies, reshape, import/export, a slicewise escape hatch, and the Lowering that
runs a graph on a MeshImpl.  Names, argument order and error types follow
mesh_tensorflow/ops.py so that code written against `mtf` reads the same
(`import mesh_amd as mtf`); the implementation is new.

Differences that matter:
  * tensors are torch tensors, dtypes are torch dtypes;
  * there is no deferred TensorFlow graph: `Lowering(graph, {mesh: impl})`
    executes each Operation's `lower` once, on the current HIP stream, and
    `Lowering.run(feeds)` executes the non-variable operations again (the
    counterpart of session.run with a feed_dict).
"""

import collections
import contextlib
import re

import numpy as np
import torch

float32 = torch.float32
bfloat16 = torch.bfloat16
int32 = torch.int32


# ----------------------------------------------------------------------------
# Dimension, Shape, layout  (mesh_tensorflow/ops.py:41-377)
# ----------------------------------------------------------------------------
Dimension = collections.namedtuple("Dimension", ["name", "size"])


def convert_to_dimension(d):
  """Dimension, (name, size) pair or None -> Dimension or None."""
  if d is None:
    return None
  if isinstance(d, Dimension):
    name, size = d.name, d.size
  else:
    name, size = d
  if not isinstance(name, str) or not isinstance(size, int):
    raise ValueError("could not convert %s to Dimension" % (d,))
  return Dimension(name, size)


class Shape(object):
  """Ordered list of uniquely named Dimensions."""

  def __init__(self, dims):
    self._dims = [convert_to_dimension(d) for d in tuple(dims)]
    names = [d.name for d in self._dims]
    if len(set(names)) != len(names):
      raise ValueError("Shape must not have repeated dimensions %s" % names)

  @property
  def dims(self):
    return list(self._dims)

  @property
  def ndims(self):
    return len(self._dims)

  @property
  def size(self):
    return list_product(self.to_integer_list)

  @property
  def to_integer_list(self):
    return [d.size for d in self._dims]

  @property
  def dimension_names(self):
    return [d.name for d in self._dims]

  @property
  def to_string(self):
    return "Shape[%s]" % ", ".join(
        "%s=%d" % (d.name, d.size) for d in self._dims)

  @property
  def cumprod(self):
    """cumprod[i] = product of the sizes of dims[i+1:] (plus a trailing 1)."""
    out, acc = [], 1
    for s in reversed(self.to_integer_list):
      out.append(acc)
      acc *= s
    return list(reversed(out))

  def __repr__(self):
    return self.to_string

  def __eq__(self, other):
    return isinstance(other, Shape) and self._dims == other._dims

  def __ne__(self, other):
    return not self == other

  def __hash__(self):
    return hash(tuple(self._dims))

  def __len__(self):
    return len(self._dims)

  def __iter__(self):
    return iter(self._dims)

  def __getitem__(self, key):
    ret = self._dims[key]
    return Shape(ret) if isinstance(key, slice) else ret

  def __add__(self, other):
    if isinstance(other, Shape):
      other = other.dims
    if isinstance(other, Dimension):
      other = [other]
    return Shape(self._dims + list(other))

  def __sub__(self, other):
    if other is None:
      return self
    if isinstance(other, Dimension):
      other = [other]
    if isinstance(other, Shape):
      other = other.dims
    return Shape([d for d in self._dims if d not in other])

  def get_dim_by_name(self, name):
    for d in self._dims:
      if d.name == name:
        return d
    raise ValueError("Dimension %s not found in %s" % (name, self.to_string))

  def rename_dimension(self, old_name, new_name):
    if old_name not in self.dimension_names:
      raise ValueError("Shape %s does not have dimension named %s"
                       % (self, old_name))
    return Shape([Dimension(new_name, d.size) if d.name == old_name else d
                  for d in self._dims])

  def resize_dimension(self, name, new_size):
    if name not in self.dimension_names:
      raise ValueError("Shape %s does not have dimension named %s"
                       % (self, name))
    return Shape([Dimension(name, new_size) if d.name == name else d
                  for d in self._dims])


def list_product(xs):
  ret = 1
  for x in xs:
    ret *= x
  return ret


def _parse_pairs(s, sep):
  """"a:b,c:d" (or with ';' / whitespace between pairs) -> [(a, b), (c, d)]."""
  pairs = []
  for item in re.split(r"[,;\s]+", s.strip()):
    if not item:
      continue
    left, right = item.split(sep)
    pairs.append((left.strip(), right.strip()))
  return pairs


def convert_to_shape(x):
  """Shape, list of Dimensions, "name:size,..." string, or None -> Shape."""
  if x is None:
    return None
  if isinstance(x, Shape):
    return x
  if isinstance(x, str):
    x = [(n, int(s)) for n, s in _parse_pairs(x, ":")]
  return Shape(x)


class LayoutRules(object):
  """Set of (tensor dimension name, mesh dimension name) pairs."""

  def __init__(self, pairs):
    self._pairs = set(tuple(p) for p in pairs)

  def __repr__(self):
    return "LayoutRules%s" % sorted(self._pairs)

  def tensor_dimension_to_mesh_axis(self, tensor_dimension, mesh_shape):
    axes = [i for i, md in enumerate(mesh_shape)
            if (tensor_dimension.name, md.name) in self._pairs]
    if len(axes) > 1:
      raise ValueError(
          "Tensor dimension maps to multiple mesh dimensions"
          " tensor_dimension=%s mesh_shape=%s layout=%s"
          % (tensor_dimension, mesh_shape, self._pairs))
    return axes[0] if axes else None

  def tensor_layout(self, tensor_shape, mesh_shape):
    axes = [self.tensor_dimension_to_mesh_axis(d, mesh_shape)
            for d in tensor_shape]
    used = [a for a in axes if a is not None]
    if len(used) != len(set(used)):
      raise ValueError(
          "Two Tensor Dimensions may not map to the same Mesh Dimension:"
          " layout=%s tensor_shape=%s mesh_shape=%s"
          % (self, tensor_shape, mesh_shape))
    return TensorLayout(axes)


class TensorLayout(object):
  """For each tensor axis, the mesh axis it is split over (or None)."""

  def __init__(self, tensor_axis_to_mesh_axis):
    self._t2m = tuple(tensor_axis_to_mesh_axis)

  @property
  def tensor_axis_to_mesh_axis(self):
    return self._t2m

  @property
  def is_fully_replicated(self):
    return all(a is None for a in self._t2m)

  def __repr__(self):
    return "TensorLayout%s" % (self._t2m,)


def convert_to_layout_rules(x):
  """LayoutRules, "tensor_dim:mesh_dim,..." string, pairs or None."""
  if isinstance(x, LayoutRules):
    return x
  if x is None:
    return LayoutRules([])
  if isinstance(x, str):
    x = _parse_pairs(x, ":")
  if isinstance(x, dict):
    x = list(x.items())
  return LayoutRules(x)


def tensor_dim_to_mesh_dim_size(layout, mesh_shape, tensor_dim):
  """How many ways `tensor_dim` is split under (layout, mesh_shape); 1 if it is
  not split (mesh_tensorflow/ops.py:6455-6477)."""
  layout_rules = convert_to_layout_rules(layout)
  mesh_shape = convert_to_shape(mesh_shape)
  if mesh_shape is None:
    return 1
  axis = layout_rules.tensor_dimension_to_mesh_axis(tensor_dim, mesh_shape)
  return 1 if axis is None else mesh_shape.dims[axis].size


# ----------------------------------------------------------------------------
# variable scopes: names only (the reference leans on tf.variable_scope)
# ----------------------------------------------------------------------------
_SCOPE_STACK = []
_REUSE_STACK = []


@contextlib.contextmanager
def variable_scope(name, reuse=None):
  """Prefixes the names of variables created inside with `name/`.  With
  reuse=True (as tf.variable_scope's, which the reference's decoding loop
  opens, transformer/transformer.py:1221) get_variable returns the existing
  variable of that name instead of creating one; the flag holds for the
  nested scopes too."""
  _SCOPE_STACK.append(name)
  _REUSE_STACK.append(bool(reuse) or (bool(_REUSE_STACK) and _REUSE_STACK[-1]))
  try:
    yield
  finally:
    _SCOPE_STACK.pop()
    _REUSE_STACK.pop()


def current_scope_name():
  return "/".join(s for s in _SCOPE_STACK if s)


# ----------------------------------------------------------------------------
# Graph, Mesh, Tensor, Operation  (mesh_tensorflow/ops.py:380-674, :841-865,
# :1423-1650)
# ----------------------------------------------------------------------------
class Graph(object):
  """Container of Operations in creation order."""

  def __init__(self):
    self._operations = []
    self._trainable_variables = []
    self._all_variables = []
    self._names = collections.Counter()

  @property
  def operations(self):
    return self._operations

  @property
  def trainable_variables(self):
    return self._trainable_variables

  @property
  def all_variables(self):
    return self._all_variables

  def unique_name(self, name):
    n = self._names[name]
    self._names[name] += 1
    return name if n == 0 else "%s_%d" % (name, n)

  def variable_by_name(self, name):
    for v in self._all_variables:
      if v.name == name:
        return v
    raise KeyError("no variable named %s (have %s)"
                   % (name, [v.name for v in self._all_variables]))


class Mesh(object):
  """A placeholder; a Lowering assigns each Mesh a MeshImpl."""

  def __init__(self, graph, name, variable_placer=None):
    self._graph = graph
    self._name = name
    self._variable_placer = variable_placer

  @property
  def graph(self):
    return self._graph

  @property
  def name(self):
    return self._name


class Tensor(object):
  """An output of an Operation: named Shape + dtype."""

  def __init__(self, operation, shape, dtype, name=None, index=0):
    if not isinstance(shape, Shape):
      raise ValueError("shape must be a Shape got %s" % (shape,))
    self._operation = operation
    self._shape = shape
    self._dtype = dtype
    self._mesh = operation.mesh
    self._name = name if name is not None else "%s:%d" % (operation.name, index)

  shape = property(lambda self: self._shape)
  size = property(lambda self: self._shape.size)
  mesh = property(lambda self: self._mesh)
  graph = property(lambda self: self._mesh.graph)
  operation = property(lambda self: self._operation)
  dtype = property(lambda self: self._dtype)
  name = property(lambda self: self._name)

  @property
  def to_string(self):
    return "Tensor[%s, %s, %s]" % (self.name, self.shape.to_string, self.dtype)

  def __repr__(self):
    return self.to_string

  def __add__(self, other):
    return add(self, other)

  def __radd__(self, other):
    return add(self, other)

  def __mul__(self, other):
    return multiply(self, other)

  def __rmul__(self, other):
    return multiply(self, other)

  def __truediv__(self, other):
    if isinstance(other, Tensor):
      raise NotImplementedError("Tensor / Tensor is not part of this subset")
    return multiply(self, 1.0 / other)


class Operation(object):
  """A node of the graph: inputs -> outputs, with a `lower` method."""

  def __init__(self, inputs, mesh=None, name=None):
    if mesh is None:
      if not inputs:
        raise ValueError("mesh must be specified if no inputs")
      mesh = inputs[0].mesh
    self._inputs = list(inputs)
    self._outputs = []
    self._mesh = mesh
    assert name is not None
    scope = current_scope_name()
    self._name = mesh.graph.unique_name(scope + "/" + name if scope else name)
    mesh.graph.operations.append(self)

  inputs = property(lambda self: self._inputs[:])
  outputs = property(lambda self: self._outputs[:])
  mesh = property(lambda self: self._mesh)
  graph = property(lambda self: self._mesh.graph)
  name = property(lambda self: self._name)

  @property
  def to_string(self):
    return "%s[Inputs=(%s) Outputs=(%s)]" % (
        type(self).__name__,
        ", ".join(t.to_string for t in self._inputs),
        ", ".join(t.to_string for t in self._outputs))

  @property
  def has_gradient(self):
    """Operations with a floating-point first output back-propagate
    (mesh_tensorflow/ops.py:1478-1482)."""
    return bool(self._outputs) and self._outputs[0].dtype.is_floating_point

  def gradient(self, unused_grad_ys):
    raise NotImplementedError(
        "Gradient not implemented for %s" % type(self).__name__)

  def lower(self, lowering):
    raise NotImplementedError("Lower not implemented")


# ----------------------------------------------------------------------------
# MeshImpl  (mesh_tensorflow/ops.py:867-1340)
# ----------------------------------------------------------------------------
class MeshImpl(object):
  """Implementation of a Mesh: mesh shape + layout rules (+ devices in
  subclasses).  Subclasses provide slicewise, the LaidOutTensor /
  LaidOutVariable types, import/export and the collectives."""

  def __init__(self, shape, layout_rules):
    self._shape = convert_to_shape(shape)
    self._layout_rules = convert_to_layout_rules(layout_rules)

  shape = property(lambda self: self._shape)
  ndims = property(lambda self: len(self._shape))
  layout_rules = property(lambda self: self._layout_rules)
  size = property(lambda self: self._shape.size)

  @property
  def supports_control_dependencies(self):
    return True

  def tensor_dimension_to_mesh_axis(self, tensor_dimension):
    return self.layout_rules.tensor_dimension_to_mesh_axis(
        tensor_dimension, self.shape)

  def tensor_layout(self, arg):
    if isinstance(arg, Tensor):
      arg = arg.shape
    return self.layout_rules.tensor_layout(arg, self.shape)

  def slice_shape(self, tensor_shape):
    """Per-device slice shape; ValueError if a mesh dim does not divide."""
    layout = self.tensor_layout(tensor_shape)
    ret = []
    for dim, axis in zip(tensor_shape, layout.tensor_axis_to_mesh_axis):
      if axis is None:
        ret.append(dim.size)
      else:
        n = self.shape[axis].size
        if dim.size % n != 0:
          raise ValueError(
              "Tensor dimension size not divisible by mesh dimension size:"
              " tensor_shape=%s tensor_layout=%s" % (tensor_shape, layout))
        ret.append(dim.size // n)
    return ret

  def slice_begin(self, tensor_shape, pnum):
    if self.size != 1:
      raise NotImplementedError("only single-device meshes are implemented")
    return [0] * tensor_shape.ndims

  def slice_size(self, tensor_shape):
    return list_product(self.slice_shape(tensor_shape))

  def laid_out_size(self, tensor_shape):
    return self.slice_size(tensor_shape) * self.size

  # -- to be provided by subclasses
  def slicewise(self, fn, *inputs):
    raise NotImplementedError("Slicewise not implemented")

  def einsum(self, equation, *slices):
    raise NotImplementedError("einsum not implemented")

  def slicewise_delay_allreduce(self, fn, *inputs):
    """slicewise that stays lazy when every input is a pending all-reduce sum
    (mesh_tensorflow/ops.py:1032-1051).  No operation of this package produces
    a pending sum (one device: nothing to reduce), so it always evaluates."""
    return self.slicewise(fn, *inputs)

  def Print(self, x, data, message, **kwargs):  # pylint: disable=invalid-name
    """The reference's default passes x through with a warning
    (mesh_tensorflow/ops.py:1053-1067); so does this."""
    del data, message, kwargs
    return x

  def allsplit(self, x, mesh_axis, split_axis, which=None):
    """Inverse of allconcat: every processor keeps the piece of its slice that
    its coordinate along mesh_axis (or `which`) names
    (mesh_tensorflow/ops.py:1082-1109)."""
    if which is None:
      which = self.laid_out_pcoord(mesh_axis)
    num_splits = self.shape[mesh_axis].size

    def keep_piece(t, w):
      piece = t.shape[split_axis] // num_splits
      return t.narrow(split_axis, int(w) * piece, piece)
    return self.slicewise(keep_piece, x, which)

  def shift_by_n_processors(self, x, mesh_axis, offset, wrap):
    """Every processor receives the slice of the one `offset` places before it
    along mesh_axis (mesh_tensorflow/ops.py:1162-1184)."""
    n = self.shape[mesh_axis].size
    source = []
    for i in range(n):
      c = i - offset
      if not 0 <= c < n:
        c = c % n if wrap else None
      source.append(c)
    return self.receive(x, mesh_axis, source)

  def laid_out_pnum(self):
    raise NotImplementedError("laid_out_pnum not implemented")

  def laid_out_pcoord(self, mesh_axis):
    """Integer scalar slices holding each processor's coordinate along
    mesh_axis (mesh_tensorflow/ops.py:1195-1210)."""
    divisor = list_product(self.shape.to_integer_list[mesh_axis + 1:])
    modulus = self.shape[mesh_axis].size
    return self.slicewise(lambda pnum: (pnum // divisor) % modulus,
                          self.laid_out_pnum())

  def laid_out_slice_num(self, tensor_shape):
    """Integer scalar slices that are equal exactly where the slices of a
    tensor of this shape are equal (mesh_tensorflow/ops.py:1212-1230)."""
    ret = self.slicewise(lambda pnum: pnum * 0, self.laid_out_pnum())
    for mesh_axis in self.tensor_layout(tensor_shape).tensor_axis_to_mesh_axis:
      if mesh_axis is not None:
        size = self.shape[mesh_axis].size
        ret = self.slicewise(lambda x, pcoord, n=size: x * n + pcoord, ret,
                             self.laid_out_pcoord(mesh_axis))
    return ret

  def broadcast_impl(self, old_slices, old_shape, new_shape):
    """Slices of old_shape -> slices of new_shape, a superset of its dimensions
    in any order (mesh_tensorflow/ops.py:1232-1247)."""
    new_slice_shape = self.slice_shape(new_shape)
    old_names = [d.name for d in old_shape.dims]
    order = [old_names.index(d.name) for d in new_shape.dims
             if d.name in old_names]
    view = [-1 if d.name in old_names else 1 for d in new_shape.dims]

    def expand(t):
      t = t.permute(order) if order else t
      sizes = iter(t.shape)
      return t.reshape([next(sizes) if v < 0 else 1 for v in view]).expand(
          new_slice_shape).contiguous()
    return self.slicewise(expand, old_slices)

  def allreduce(self, x, mesh_axes, reduction_fn_string):
    raise NotImplementedError("Allreduce not implemented")

  def allconcat(self, x, mesh_axis, concat_axis):
    raise NotImplementedError("Allconcat not implemented")

  def alltoall(self, x, mesh_axis, split_axis, concat_axis):
    raise NotImplementedError("Alltoall not implemented")

  def receive(self, x, mesh_axis, source_pcoord):
    raise NotImplementedError("Receive not implemented")

  def import_tf_tensor(self, x, tf_x):
    raise NotImplementedError("Import not implemented")

  def export_to_tf_tensor(self, x, laid_out_x):
    raise NotImplementedError("Export not implemented")

  def make_slices(self, tf_tensor, tensor_shape):
    if self.size != 1:
      raise NotImplementedError("only single-device meshes are implemented")
    return [tf_tensor]

  def combine_slices(self, slices, tensor_shape, device=None):
    if self.size != 1:
      raise NotImplementedError("only single-device meshes are implemented")
    return slices[0]


def convert_args_to_laid_out_tensors(xs):
  """Calls to_laid_out_tensor() on the arguments that have it."""
  return [x.to_laid_out_tensor() if hasattr(x, "to_laid_out_tensor") else x
          for x in xs]


# ----------------------------------------------------------------------------
# Lowering  (mesh_tensorflow/ops.py:676-838)
# ----------------------------------------------------------------------------
class Lowering(object):
  """Runs a Graph on MeshImpls.

  Construction lowers (= executes) every Operation once, in graph order.
  `run(feeds)` executes them again without re-creating variables.
  """

  def __init__(self, graph, mesh_to_impl, autostack=True, log_file=None,
               initial_values=None):
    del autostack, log_file  # accepted for signature compatibility
    self.mesh_to_impl = mesh_to_impl
    self.graph = graph
    self._counters = []
    self.tensors = {}      # {Tensor: LaidOutTensor}
    self.operations = {}   # {Operation: lowered handle}
    self.variables = {}    # {Variable: LaidOutVariable}
    self.initial_values = dict(initial_values or {})
    self._feeds = {}
    self.scalar_summaries = {}   # {name: 0-d torch tensor} of the last run
    for op in graph.operations:
      op.lower(self)
      for out in op.outputs:
        self.add_counter("output/%s" % type(op).__name__,
                         self.laid_out_size(out))
        self.add_counter("output_unique/%s" % type(op).__name__, out.size)

  def run(self, feeds=None):
    """Executes the graph's non-variable operations again.  `feeds` maps
    imported Tensors to new torch tensors of the same shape."""
    self._feeds = dict(feeds or {})
    self.scalar_summaries = {}
    try:
      for op in self.graph.operations:
        if not isinstance(op, Variable):
          op.lower(self)
    finally:
      self._feeds = {}

  def fed_value(self, tensor, default):
    return self._feeds.get(tensor, default)

  def capture(self):
    """Records one `run()` into a HIP graph and returns a CapturedStep whose
    `replay(feeds)` re-executes it with one graph launch instead of one launch
    per kernel (what pays when the step is launch-bound: small layers).

    Every imported tensor gets a static device buffer that the recorded
    kernels read; `replay` copies new values into those buffers first.  The
    outputs live in the graph's memory pool: `export_to_tf_tensor` returns the
    tensors the last replay wrote.  Variables are read in place and
    LaidOutVariable updates its master, slice and packed copies in place
    (assign, assign_to_slices, copy_master_to_slices, a checkpoint restore),
    so an assignment between replays is seen.  The library allocates nothing
    and uses no memset nodes, which is what makes its launches capturable.
    """
    statics = {}
    for op in self.graph.operations:
      if isinstance(op, ImportOperation):
        t = op.outputs[0]
        statics[t] = self.tensors[t].to_laid_out_tensor().tensor_list[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):     # warm-up outside the capture
      self.run(statics)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      self.run(statics)
    return CapturedStep(graph, statics, self, dict(self.tensors))

  def mesh_impl(self, m):
    if not isinstance(m, Mesh):
      m = m.mesh
    return self.mesh_to_impl[m]

  def export_to_tf_tensor(self, x):
    """Tensor -> torch tensor (the name is the reference's)."""
    mesh_impl = self.mesh_impl(x)
    return mesh_impl.export_to_tf_tensor(
        x, self.tensors[x].to_laid_out_tensor())

  export_to_torch = export_to_tf_tensor

  def lowered_operation(self, op):
    return self.operations[op]

  def copy_masters_to_slices(self):
    for v in self.variables.values():
      v.copy_master_to_slices()

  def copy_slices_to_masters(self):
    for v in self.variables.values():
      v.copy_slices_to_master()

  def add_scalar_summary(self, name, value):
    """Records a 0-d device tensor under `name` for this run (what
    tf.summary.scalar does with the reference's ScalarSummaryOperation,
    ops.py:4402-4436).  A name used before in the same run gets the suffix
    _1, _2, .. as TensorFlow's summary names do."""
    key, n = name, 0
    while key in self.scalar_summaries:
      n += 1
      key = "%s_%d" % (name, n)
    self.scalar_summaries[key] = value.reshape(())

  def add_counter(self, key, value):
    assert isinstance(value, int)
    self._counters.append((key, value))

  @property
  def counters(self):
    return self._counters

  def laid_out_size(self, tensor):
    return self.mesh_impl(tensor).laid_out_size(tensor.shape)

  def set_tensor_lowering(self, tensor, laid_out_tensor):
    self.verify_slice_shapes(tensor, laid_out_tensor)
    self.tensors[tensor] = laid_out_tensor

  def verify_slice_shapes(self, tensor, laid_out_tensor):
    correct_shape = self.mesh_impl(tensor).slice_shape(tensor.shape)
    actual_shape = list(laid_out_tensor.slice_shape)
    if actual_shape != correct_shape:
      raise ValueError(
          "Wrong slice shape: correct_shape = %s actual shape = %s"
          % (correct_shape, actual_shape))


class CapturedStep(object):
  """A recorded step of a Lowering (Lowering.capture)."""

  def __init__(self, graph, statics, lowering, recorded_tensors):
    self._graph = graph
    self._statics = statics
    self._lowering = lowering
    self._recorded = recorded_tensors

  def replay(self, feeds=None):
    """feeds: {imported Tensor: torch tensor of the same shape}; tensors not
    fed keep the values of the previous replay."""
    for tensor, value in (feeds or {}).items():
      if tensor not in self._statics:
        raise ValueError("%s is not an imported tensor of the recorded graph"
                         % (tensor,))
      self._statics[tensor].copy_(torch.as_tensor(value))
    self._graph.replay()
    # an eager run() since the capture has rebound the lowering's tensors to
    # its own results: point them back at what the recorded kernels write
    self._lowering.tensors.update(self._recorded)


# ----------------------------------------------------------------------------
# operations
# ----------------------------------------------------------------------------
class SlicewiseOperation(Operation):
  """Applies a torch function to the slices (mesh_tensorflow/ops.py:1651-1723).
  `tf_fn` maps input slices to one output slice or a tuple of them."""

  def __init__(self, tf_fn, inputs, output_shapes, output_dtypes,
               splittable_dims=None, grad_function=None, name=None):
    super(SlicewiseOperation, self).__init__(inputs, name=name or "slicewise")
    del splittable_dims
    self._grad_function = grad_function
    self._tf_fn = tf_fn
    self._outputs = [Tensor(self, convert_to_shape(s), d, index=i)
                     for i, (s, d) in enumerate(zip(output_shapes,
                                                    output_dtypes))]

  @property
  def has_gradient(self):
    return self._grad_function is not None

  def gradient(self, grad_ys):
    # the reference calls grad_function(op, *grad_ys) (ops.py:1705-1708)
    return self._grad_function(self, *grad_ys)

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    values = mesh_impl.slicewise(
        self._tf_fn, *[lowering.tensors[x] for x in self.inputs])
    if len(self.outputs) == 1 and not isinstance(values, tuple):
      values = (values,)
    for out, v in zip(self.outputs, values):
      lowering.set_tensor_lowering(out, v)


def slicewise(tf_fn, xs, output_shape=None, output_dtype=None,
              splittable_dims=None, grad_function=None, name=None):
  """mtf.slicewise (mesh_tensorflow/ops.py:1726-1763)."""
  multiple = isinstance(output_shape, list)
  shapes = output_shape if multiple else [output_shape or xs[0].shape]
  dtypes = output_dtype if multiple else [output_dtype or xs[0].dtype]
  outs = SlicewiseOperation(tf_fn, xs, shapes, dtypes, splittable_dims,
                            grad_function, name=name).outputs
  return tuple(outs) if multiple else outs[0]


def cwise(tf_fn, xs, output_dtype=None, grad_function=None, name=None):
  return slicewise(tf_fn, xs, output_dtype=output_dtype,
                   grad_function=grad_function, name=name or "cwise")


def cast(x, dtype, name="cast"):
  if dtype == x.dtype:
    return x
  # the gradient of a cast casts back (mesh_tensorflow/ops.py:1945-1962)
  return cwise(lambda t: t.to(dtype), [x], output_dtype=dtype, name=name,
               grad_function=lambda op, dy: [cast(dy, op.inputs[0].dtype)])


def not_equal(x, value, name="not_equal"):
  """x != a Python scalar, as a bool tensor (mesh_tensorflow/ops.py:2121-2123
  for this case)."""
  if isinstance(value, Tensor):
    raise NotImplementedError("not_equal of two Tensors")
  return cwise(lambda t: t != value, [x], output_dtype=torch.bool, name=name)


def to_float(x, name="to_float"):
  return cast(x, float32, name=name)


def to_bfloat16(x, name="to_bfloat16"):
  return cast(x, bfloat16, name=name)


def _scalar_in(dtype, value):
  """A Python scalar as the reference's scalar ops see it: rounded to the
  tensor's dtype first."""
  return torch.tensor(value, dtype=dtype).item()


def add(x1, x2, output_shape=None, name=None):
  """Tensor + scalar, or Tensor + Tensor with broadcasting of x2's dims that
  are a subsequence of x1's (all the MoE layers need)."""
  del output_shape
  if not isinstance(x2, Tensor):
    c = _scalar_in(x1.dtype, x2)
    return cwise(lambda t: t + c, [x1], name=name or "scalar_add",
                 grad_function=lambda op, dy: [dy])
  if not isinstance(x1, Tensor):
    return add(x2, x1)
  big, small = (x1, x2) if x1.shape.ndims >= x2.shape.ndims else (x2, x1)
  names = big.shape.dimension_names
  if any(d not in big.shape.dims for d in small.shape.dims):
    raise ValueError("cannot broadcast %s to %s" % (small.shape, big.shape))
  view = [d.size if d in small.shape.dims else 1 for d in big.shape.dims]
  order = [names.index(d.name) for d in small.shape.dims]
  if order != sorted(order):
    raise ValueError("dimension order differs: %s vs %s"
                     % (small.shape, big.shape))

  def fn(a, b):
    return a + b.reshape(view).to(a.dtype)
  grad = None
  if big.shape == small.shape and big.dtype == small.dtype:
    grad = lambda op, dy: [dy, dy]     # what accumulating gradients needs
  return slicewise(fn, [big, small], output_shape=big.shape,
                   output_dtype=big.dtype, name=name or "add",
                   grad_function=grad)


def multiply(x1, x2, output_shape=None, name=None):
  """Tensor * Python scalar (ScalarMultiplyOperation,
  mesh_tensorflow/ops.py:2006-2023), or Tensor * Tensor where the dims of the
  smaller one are a subsequence of the larger one's (mtf.multiply's
  broadcasting, mesh_tensorflow/ops.py:5135-5153).  Both operands get a
  gradient, as in the reference (BinaryOpWithBroadcasting's gradient,
  ops.py:2044-2084): d(big) = dy * small, d(small) = dy * big summed over the
  dims the small operand does not have (float32 accumulation, one rounding to
  the small operand's dtype)."""
  del output_shape
  if isinstance(x2, Tensor) and not isinstance(x1, Tensor):
    x1, x2 = x2, x1
  if isinstance(x2, Tensor):
    big, small = (x1, x2) if x1.shape.ndims >= x2.shape.ndims else (x2, x1)
    names = big.shape.dimension_names
    if any(d not in big.shape.dims for d in small.shape.dims):
      raise ValueError("cannot broadcast %s to %s" % (small.shape, big.shape))
    order = [names.index(d.name) for d in small.shape.dims]
    if order != sorted(order):
      raise ValueError("dimension order differs: %s vs %s"
                       % (small.shape, big.shape))
    view = [d.size if d in small.shape.dims else 1 for d in big.shape.dims]

    def fn(a, b):
      return a * b.reshape(view).to(a.dtype)

    reduced = [i for i, d in enumerate(big.shape.dims)
               if d not in small.shape.dims]
    small_sizes = small.shape.to_integer_list

    def small_grad_fn(dy, a):
      prod = dy.to(torch.float32) * a.to(torch.float32)
      if reduced:
        prod = prod.sum(dim=reduced)
      return prod.reshape(small_sizes).to(small.dtype)

    def grad(op, dy):
      # (a mask or another constant of the graph needs none: no reduction
      # over the activations is built for it)
      d_small = None
      if _gradient_wanted(op.inputs[1]):
        d_small = slicewise(small_grad_fn, [dy, op.inputs[0]],
                            output_shape=small.shape, output_dtype=small.dtype,
                            name="mul_grad_small")
      return [multiply(dy, op.inputs[1]), d_small]
    return slicewise(
        fn, [big, small], output_shape=big.shape, output_dtype=big.dtype,
        name=name or "mul", grad_function=grad)
  c = _scalar_in(x1.dtype, x2)
  return cwise(lambda t: t * c, [x1], name=name or "scalar_mul",
               grad_function=lambda op, dy: [multiply(dy, x2)])


class ScalarSummaryOperation(Operation):
  """mtf.scalar_summary (ops.py:4402-4436): passes x through and records its
  value under `name` on the Lowering (Lowering.scalar_summaries)."""

  def __init__(self, name, x):
    super(ScalarSummaryOperation, self).__init__(
        [x], x.mesh, name=name + "_summary")
    if x.shape.dims:
      raise ValueError("ScalarSummaryOperation takes a scalar")
    self._summary_name = name
    self._outputs = [Tensor(self, x.shape, x.dtype)]

  def gradient(self, grad_ys):
    return grad_ys

  def lower(self, lowering):
    x = lowering.tensors[self.inputs[0]]
    lowering.add_scalar_summary(
        self._summary_name, x.to_laid_out_tensor().tensor_list[0])
    lowering.set_tensor_lowering(self.outputs[0], x)


def scalar_summary(name, x):
  """Records the 0-dimensional Tensor x under `name`; returns a Tensor equal
  to x (ops.py:4423-4436)."""
  return ScalarSummaryOperation(name, x).outputs[0]


class ReshapeOperation(Operation):
  """Reshape to a Shape of equal size (mesh_tensorflow/ops.py:4477-4580); on a
  single device this is a view."""

  def __init__(self, x, new_shape, name=None):
    super(ReshapeOperation, self).__init__([x], name=name or "reshape")
    if x.shape.size != new_shape.size:
      raise ValueError("Cannot reshape Tensor %s to shape %s - sizes differ."
                       % (x, new_shape))
    self._outputs = [Tensor(self, new_shape, x.dtype)]

  def gradient(self, grad_ys):
    return [reshape(grad_ys[0], self.inputs[0].shape)]

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    new_shape = self.outputs[0].shape
    if mesh_impl.size != 1:
      raise NotImplementedError("reshape across a split mesh dimension")
    sizes = new_shape.to_integer_list
    lowering.set_tensor_lowering(
        self.outputs[0],
        mesh_impl.slicewise(lambda t: t.reshape(sizes),
                            lowering.tensors[self.inputs[0]]))


def reshape(x, new_shape, name="reshape"):
  new_shape = convert_to_shape(new_shape)
  if new_shape == x.shape:
    return x
  return ReshapeOperation(x, new_shape, name=name).outputs[0]


def rename_dimension(x, old_name, new_name):
  return reshape(x, x.shape.rename_dimension(old_name, new_name))


class ImportOperation(Operation):
  """Brings a torch tensor into the graph (mesh_tensorflow/ops.py:3854-3875)."""

  def __init__(self, mesh, tf_tensor, shape, name=None):
    super(ImportOperation, self).__init__([], mesh=mesh, name=name or "import")
    tf_tensor = torch.as_tensor(tf_tensor)
    if list(tf_tensor.shape) != shape.to_integer_list:
      raise ValueError("Incompatible shape; have %s, want %s"
                       % (list(tf_tensor.shape), shape))
    self._outputs = [Tensor(self, shape, tf_tensor.dtype)]
    self._tf_tensor = tf_tensor

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    value = lowering.fed_value(self.outputs[0], self._tf_tensor)
    lowering.set_tensor_lowering(
        self.outputs[0], mesh_impl.import_tf_tensor(self.outputs[0], value))


def import_tf_tensor(mesh, tf_tensor, shape=None, name=None):
  """Torch tensor (or array) -> Tensor.  The name is the reference's."""
  tf_tensor = torch.as_tensor(tf_tensor)
  if shape is None:
    shape = Shape([Dimension("anon_%d" % i, int(s))
                   for i, s in enumerate(tf_tensor.shape)])
  return ImportOperation(mesh, tf_tensor, convert_to_shape(shape),
                         name=name).outputs[0]


import_tensor = import_tf_tensor


class Constant(Operation):
  """A tensor filled with one value (mesh_tensorflow/ops.py:4337-4355)."""

  def __init__(self, mesh, value, shape, dtype, name=None):
    super(Constant, self).__init__([], mesh, name=name or "constant")
    self._outputs = [Tensor(self, shape, dtype)]
    self._value = value

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    out = self.outputs[0]
    sizes = mesh_impl.slice_shape(out.shape)
    lowering.set_tensor_lowering(
        out, mesh_impl.slicewise(
            lambda: torch.full(sizes, self._value, dtype=out.dtype,
                               device=mesh_impl.device)))


def constant(mesh, value, shape=None, dtype=float32):
  return Constant(mesh, value, convert_to_shape(shape or []), dtype).outputs[0]


def zeros(mesh, shape, dtype=float32):
  return constant(mesh, 0, shape=convert_to_shape(shape), dtype=dtype)


class VariableDType(object):
  """master / slice / activation dtypes of a variable
  (mesh_tensorflow/ops.py:3961-4003)."""

  def __init__(self, master_dtype=float32, slice_dtype=None,
               activation_dtype=None):
    self._master_dtype = master_dtype
    self._slice_dtype = slice_dtype or master_dtype
    self._activation_dtype = activation_dtype or master_dtype

  master_dtype = property(lambda self: self._master_dtype)
  slice_dtype = property(lambda self: self._slice_dtype)
  activation_dtype = property(lambda self: self._activation_dtype)


class Variable(Operation):
  """A named parameter (mesh_tensorflow/ops.py:4006-4093).  Lowering creates a
  LaidOutVariable; its output is the slice cast to the activation dtype,
  produced lazily so that consumers with their own packed copy never pay for
  the cast."""

  def __init__(self, mesh, name, shape, dtype, initializer, trainable,
               **kwargs):
    del kwargs
    super(Variable, self).__init__([], mesh, name=name)
    if not isinstance(dtype, VariableDType):
      raise ValueError("dtype must be a VariableDType got %s" % dtype)
    self._dtype = dtype
    self._trainable = trainable
    self._initializer = initializer
    self._outputs = [Tensor(self, shape, dtype.activation_dtype)]
    self.graph.all_variables.append(self)
    if trainable:
      self.graph.trainable_variables.append(self)

  def __repr__(self):
    return "Variable(%s)" % self.value

  value = property(lambda self: self.outputs[0])
  shape = property(lambda self: self.value.shape)
  dtype = property(lambda self: self._dtype)
  master_dtype = property(lambda self: self._dtype.master_dtype)
  slice_dtype = property(lambda self: self._dtype.slice_dtype)
  activation_dtype = property(lambda self: self._dtype.activation_dtype)
  trainable = property(lambda self: self._trainable)
  initializer = property(lambda self: self._initializer)

  def lower(self, lowering):
    mesh_impl = lowering.mesh_impl(self)
    initial = lowering.initial_values.get(self.name)
    sv = mesh_impl.LaidOutVariable(self, mesh_impl, initial_value=initial)
    lowering.variables[self] = sv
    lowering.set_tensor_lowering(self.outputs[0], sv.activation_tensor())
    key = "variables/trainable" if self._trainable else "variables/untrainable"
    lowering.add_counter(key, self.outputs[0].size)


def get_variable(mesh, name, shape, dtype=float32, master_dtype=None,
                 slice_dtype=None, activation_dtype=None, initializer=None,
                 trainable=True, **kwargs):
  """Creates a variable named `<scope>/<name>`
  (mesh_tensorflow/ops.py:4160-4208); inside variable_scope(..., reuse=True)
  returns the existing one.  Asking for an existing name without reuse
  raises."""
  if dtype is None:
    dtype = VariableDType(master_dtype, slice_dtype, activation_dtype)
  elif isinstance(dtype, VariableDType):
    if master_dtype or slice_dtype or activation_dtype:
      raise ValueError("dtype is a VariableDType; do not also pass its parts")
  else:
    dtype = VariableDType(master_dtype or dtype, slice_dtype or dtype,
                          activation_dtype or dtype)
  scope = current_scope_name()
  full = scope + "/" + name if scope else name
  existing = [v for v in mesh.graph.all_variables if v.name == full]
  if _REUSE_STACK and _REUSE_STACK[-1]:
    if not existing:
      raise ValueError("Variable %s does not exist (reuse=True)" % full)
    out = existing[0].outputs[0]
    if out.shape != convert_to_shape(shape):
      raise ValueError("Variable %s has shape %s, asked for %s"
                       % (full, out.shape, convert_to_shape(shape)))
    return out
  if existing:
    raise ValueError("Variable %s already exists" % full)
  return Variable(mesh, name, convert_to_shape(shape), dtype, initializer,
                  trainable, **kwargs).outputs[0]


# While gradients() walks the graph: the tensors that depend on one of its
# `xs` (only those are given a gradient); None outside it.
_GRADIENT_TARGETS = None
_GRADIENT_XS = None     # the `xs` themselves


def gradient_is_returned(tensor):
  """Inside an Operation.gradient call: is `tensor` one of the tensors whose
  gradient gradients() hands back to its caller (who must then see the true
  derivative, not a fused form meant for one particular consumer)?"""
  return _GRADIENT_XS is None or tensor in _GRADIENT_XS


def _gradient_wanted(tensor):
  """Inside an Operation.gradient call: does gradients() keep a gradient for
  `tensor`?  (Outside gradients(): unknown, so yes.)"""
  return _GRADIENT_TARGETS is None or tensor in _GRADIENT_TARGETS


def gradients(ys, xs, grad_ys=None, operations=None):
  """mtf.gradients (mesh_tensorflow/ops.py:5254-5291): gradient Tensors of the
  sum of `ys` (weighted by grad_ys) w.r.t. each of `xs`, built by walking the
  graph backwards and calling Operation.gradient.  None for an x nothing
  depends on."""
  if operations is None:
    operations = ys[0].graph.operations
  if not grad_ys:
    grad_ys = [Constant(y.mesh, 1.0, y.shape, y.dtype).outputs[0] for y in ys]
  downstream = set(xs)
  for op in operations:
    if op.has_gradient:
      if set(op.inputs) & downstream:
        downstream |= set(op.outputs)
  tensor_to_gradient = {y: g for y, g in zip(ys, grad_ys) if g is not None}
  global _GRADIENT_TARGETS, _GRADIENT_XS
  outer_targets, _GRADIENT_TARGETS = _GRADIENT_TARGETS, downstream
  outer_xs, _GRADIENT_XS = _GRADIENT_XS, set(xs)
  try:
    for op in operations[::-1]:
      grad_outputs = [tensor_to_gradient.get(out) for out in op.outputs]
      if (op.has_gradient and any(g is not None for g in grad_outputs)
          and (set(op.inputs) & downstream)):
        with variable_scope(op.name + "/gradients"):
          input_grads = op.gradient(grad_outputs)
          for inp, grad in zip(op.inputs, input_grads):
            if inp in downstream and grad is not None:
              if inp in tensor_to_gradient:
                tensor_to_gradient[inp] = tensor_to_gradient[inp] + grad
              else:
                tensor_to_gradient[inp] = grad
  finally:
    _GRADIENT_TARGETS = outer_targets
    _GRADIENT_XS = outer_xs
  return [tensor_to_gradient.get(x, None) for x in xs]


def relu(x, name="relu"):
  return cwise(torch.relu, [x], name=name)


def _dropout_sizes(shape, noise_shape):
  """x's dimensions as (outer, mid, inner) sizes, `mid` covering the one run of
  consecutive dimensions that noise_shape leaves out."""
  missing = [d for d in noise_shape.dims if d not in shape.dims]
  if missing:
    raise ValueError("noise_shape %s is not a subset of %s"
                     % (noise_shape, shape))
  flags = [d in noise_shape.dims for d in shape.dims]
  if [d for d in shape.dims if d in noise_shape.dims] != noise_shape.dims:
    raise NotImplementedError(
        "dropout noise_shape %s orders its dimensions differently from %s"
        % (noise_shape, shape))
  if all(flags):
    return 1, 1, shape.size
  first = flags.index(False)
  last = len(flags) - 1 - flags[::-1].index(False)
  if any(flags[first:last + 1]):
    raise NotImplementedError(
        "dropout noise broadcast over dimensions of %s that are not "
        "consecutive (noise_shape %s)" % (shape, noise_shape))
  sizes = shape.to_integer_list
  return (list_product(sizes[:first]), list_product(sizes[first:last + 1]),
          list_product(sizes[last + 1:]))


class DropoutOperation(Operation):
  """x * noise, noise = (uniform < keep_prob) / keep_prob drawn in x's dtype
  over noise_shape and broadcast over x's other dimensions
  (mesh_tensorflow/ops.py:5832-5872).  The uniform numbers come from torch's
  generator on the device, or from `uniform` (a tensor of outer * inner
  elements) when it is set before lowering; `noise` holds the multiplier of
  the last lowering."""

  def __init__(self, x, keep_prob, noise_shape, name=None):
    # checked first: a constructor that raises must not leave its operation
    # in the graph
    self.sizes = _dropout_sizes(x.shape, noise_shape)
    super(DropoutOperation, self).__init__([x], name=name or "dropout")
    self.keep_prob = keep_prob
    self.noise_shape = noise_shape
    self._outputs = [Tensor(self, x.shape, x.dtype)]
    self.uniform = None
    self.noise = None

  def gradient(self, grad_ys):
    return [DropoutGradOperation(self, grad_ys[0]).outputs[0]]

  def lower(self, lowering):
    from mesh_amd import moe_hip  # pylint: disable=g-import-not-at-top
    outer, _, inner = self.sizes

    def fn(t):
      u = self.uniform
      if u is None:
        u = torch.rand((outer, inner), dtype=t.dtype, device=t.device)
      out, self.noise = moe_hip.broadcast_dropout(
          t.contiguous(), self.sizes, uniform=u.to(t.dtype).contiguous(),
          keep_prob=self.keep_prob, want_noise=True)
      return out
    lowering.set_tensor_lowering(
        self.outputs[0], lowering.mesh_impl(self).slicewise(
            fn, lowering.tensors[self.inputs[0]]))


class DropoutGradOperation(Operation):
  """dx = dy * noise with the multiplier the forward lowering drew."""

  def __init__(self, forward, dy, name=None):
    super(DropoutGradOperation, self).__init__(
        [dy, forward.outputs[0]], name=name or "dropout_grad")
    self._forward = forward
    self._outputs = [Tensor(self, dy.shape, dy.dtype)]

  def lower(self, lowering):
    from mesh_amd import moe_hip  # pylint: disable=g-import-not-at-top
    forward = self._forward

    def fn(dy, unused_y):
      return moe_hip.broadcast_dropout(dy.contiguous(), forward.sizes,
                                       noise=forward.noise)[0]
    lowering.set_tensor_lowering(
        self.outputs[0], lowering.mesh_impl(self).slicewise(
            fn, *[lowering.tensors[x] for x in self.inputs]))


def dropout(x, is_training, keep_prob=None, rate=None, noise_shape=None,
            name=None):
  """mtf.dropout (mesh_tensorflow/ops.py:5832-5872): identity unless training;
  kept elements are scaled by 1 / keep_prob."""
  if (keep_prob is None) == (rate is None):
    raise ValueError("exactly one of keep_prob and rate should be set")
  if keep_prob is None:
    keep_prob = 1.0 - rate
  noise_shape = convert_to_shape(noise_shape)
  if noise_shape is None:
    noise_shape = x.shape
  if keep_prob == 1.0 or not is_training:
    return x
  if not x.dtype.is_floating_point:
    raise NotImplementedError("dropout of an integer tensor")
  return DropoutOperation(x, keep_prob, noise_shape, name=name).outputs[0]


def to_numpy(t):
  """Torch tensor -> float32/int NumPy array on the host."""
  t = t.detach()
  if t.dtype == torch.bfloat16:
    t = t.float()
  return np.asarray(t.cpu())
