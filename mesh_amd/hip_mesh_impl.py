"""HipMeshImpl: a single-device MeshImpl whose slices are torch tensors in the
HBM of one MI355X and whose Mixture-of-Experts operations run on
libmesh_moe_hip.so.

It plays the role PlacementMeshImpl(shape=[], layout={}, devices=[""]) plays in
the reference (mesh_tensorflow/placement_mesh_impl.py:31-355,
mesh_tensorflow/test_utils.py:54-55): one slice per tensor, collectives that
return their input (placement_mesh_impl.py:291-292, :376-377).
"""

import torch

from mesh_amd import moe_hip
from mesh_amd import ops as mtf


class HipMeshImpl(mtf.MeshImpl):
  """Mesh implementation for one GPU."""

  def __init__(self, shape=None, layout=None, devices=None, device=None):
    """Args mirror PlacementMeshImpl(shape, layout, devices); only the empty
    mesh shape (one device) is supported.  `device` (or devices[0]) names the
    torch device; "" or None means the current GPU."""
    super(HipMeshImpl, self).__init__(shape if shape is not None else [],
                                      layout if layout is not None else {})
    if self.size != 1:
      raise ValueError("HipMeshImpl runs on one GPU: mesh shape %s has %d "
                       "processors" % (self.shape, self.size))
    if devices is not None and len(devices) != 1:
      raise ValueError("HipMeshImpl takes exactly one device, got %s"
                       % (devices,))
    if device is None and devices:
      device = devices[0] or None
    if not torch.cuda.is_available():
      raise RuntimeError(
          "HipMeshImpl needs a GPU: torch.cuda.is_available() is False "
          "(there is no CPU path)")
    self._device = torch.device(device or "cuda:%d" % torch.cuda.current_device())
    moe_hip.load_library()  # fail now, not at the first kernel, if not built

  device = property(lambda self: self._device)
  devices = property(lambda self: [str(self._device)])

  class LaidOutTensor(object):
    """One slice per processor; here always exactly one."""

    def __init__(self, tensor_list):
      self._tensor_list = list(tensor_list)

    def __repr__(self):
      return "[" + ",".join(str(tuple(t.shape)) for t in self._tensor_list) + "]"

    tensor_list = property(lambda self: self._tensor_list)
    all_slices = property(lambda self: self._tensor_list)

    @classmethod
    def from_tensor_list(cls, tensor_list):
      return cls(tensor_list)

    @property
    def slice_shape(self):
      return list(self._tensor_list[0].shape)

    def to_laid_out_tensor(self):
      return self

  class LazyLaidOutTensor(object):
    """A LaidOutTensor computed on first use (the reference has the same idea,
    mesh_tensorflow/ops.py:3941-3958)."""

    def __init__(self, thunk, slice_shape):
      self._thunk = thunk
      self._slice_shape = list(slice_shape)

    slice_shape = property(lambda self: self._slice_shape)

    def to_laid_out_tensor(self):
      return self._thunk()

  class LaidOutVariable(object):
    """Master copy, slice copy and derived read-only copies of one variable
    (mesh_tensorflow/placement_mesh_impl.py:67-157).

    master: master_dtype, what checkpoints hold; slice: slice_dtype, what the
    optimizer would update.  With equal dtypes on one device the slice is the
    master (placement_mesh_impl.py:119-130).  `packed(dtype)` is the
    K-contiguous activation-dtype copy the expert GEMM reads; it is rebuilt
    when the slice changes.
    """

    def __init__(self, variable, mesh_impl, initial_value=None):
      self._variable = variable
      self._mesh_impl = mesh_impl
      shape = variable.shape.to_integer_list
      dev = mesh_impl.device
      if initial_value is None:
        init = variable.initializer
        if init is None:
          raise ValueError("variable %s has no initializer and no initial "
                           "value" % variable.name)
        initial_value = init
      if callable(initial_value):
        initial_value = initial_value(shape, variable.master_dtype, dev)
      master = torch.as_tensor(initial_value)
      if list(master.shape) != shape:
        raise ValueError("initial value of %s has shape %s, want %s"
                         % (variable.name, list(master.shape), shape))
      self._master = master.to(device=dev, dtype=variable.master_dtype).contiguous()
      self._slice = None
      self._derived = {}
      self.copy_master_to_slices()

    variable = property(lambda self: self._variable)
    master = property(lambda self: self._master)

    @property
    def laid_out_tensor(self):
      return self._mesh_impl.LaidOutTensor([self._slice])

    @property
    def slice_shape(self):
      return list(self._slice.shape)

    # Every update below writes into the storage that already exists: a step
    # recorded into a HIP graph (Lowering.capture) holds the device addresses
    # of the slice and of its derived copies, and must see the new values.

    def copy_master_to_slices(self):
      v = self._variable
      if v.slice_dtype == v.master_dtype:
        self._slice = self._master
      elif self._slice is None:
        self._slice = self._master.to(v.slice_dtype)
      else:
        self._slice.copy_(self._master)
      self._refresh_derived()

    def copy_slices_to_master(self):
      if self._master is not self._slice:
        self._master.copy_(self._slice)

    def assign_to_slices(self, assign_fn, values, assign_to_tensor_list=None):
      del assign_fn, assign_to_tensor_list
      (value,) = values
      self._slice.copy_(value)
      self._refresh_derived()

    def assign(self, value):
      """Sets master and slice from an array / tensor (replaces TF
      initialisers and checkpoint restore)."""
      v = self._variable
      value = torch.as_tensor(value)
      if list(value.shape) != v.shape.to_integer_list:
        raise ValueError("value for %s has shape %s, want %s"
                         % (v.name, list(value.shape), v.shape.to_integer_list))
      self._master.copy_(value)
      self.copy_master_to_slices()

    def _refresh_derived(self):
      """Recomputes the derived copies of the slice in place."""
      for (kind, dtype), t in self._derived.items():
        if kind == "act":
          t.copy_(self._slice)
        else:
          s = self._slice
          moe_hip.pack_weights(s.reshape(-1, s.shape[-2], s.shape[-1]), dtype,
                               out=t)

    def activation_tensor(self):
      """Slice cast to the activation dtype (Variable.lower,
      mesh_tensorflow/ops.py:4039-4047), computed on demand and cached."""
      def thunk():
        key = ("act", self._variable.activation_dtype)
        if key not in self._derived:
          self._derived[key] = self._slice.to(self._variable.activation_dtype)
        return self._mesh_impl.LaidOutTensor([self._derived[key]])
      return self._mesh_impl.LazyLaidOutTensor(thunk, self.slice_shape)

    def packed(self, dtype):
      """[..., K, N] slice -> [E, N, K] of `dtype` (leading dims flattened into
      E), the layout mesh_moe_expert_ffn reads."""
      key = ("packed", dtype)
      if key not in self._derived:
        s = self._slice
        k, n = s.shape[-2], s.shape[-1]
        self._derived[key] = moe_hip.pack_weights(s.reshape(-1, k, n), dtype)
      return self._derived[key]

  # -- execution -------------------------------------------------------------
  def slicewise(self, fn, *inputs):
    """Calls fn once on the single slice of each input
    (mesh_tensorflow/placement_mesh_impl.py:159-178)."""
    inputs = mtf.convert_args_to_laid_out_tensors(inputs)
    args = [x.tensor_list[0] if isinstance(x, self.LaidOutTensor) else x
            for x in inputs]
    with torch.cuda.device(self._device):
      ret = fn(*args)
    if isinstance(ret, tuple):
      return tuple(self.LaidOutTensor([t]) for t in ret)
    return self.LaidOutTensor([ret])

  def einsum(self, equation, *slices):
    """The hook the reference documents "for custom einsum implementation"
    (mesh_tensorflow/ops.py:1331-1340; its default is tf.einsum).  Called with
    the slices themselves, from inside a slice function.  The layers of this
    package do not come through here: their contractions run on the library's
    kernels; this serves Operations written against the reference interface."""
    return torch.einsum(equation, *slices)

  def laid_out_pnum(self):
    """Processor number: one int32 scalar slice, 0
    (mesh_tensorflow/placement_mesh_impl.py:327-329, where the
    slices are Python ints; here a device tensor, like every other slice)."""
    return self.LaidOutTensor(
        [torch.zeros((), dtype=torch.int32, device=self._device)])

  # collectives on one processor return their input
  def allreduce(self, x, mesh_axes, reduction_fn_string):
    return x

  def allconcat(self, x, mesh_axis, concat_axis):
    return x

  def alltoall(self, x, mesh_axis, split_axis, concat_axis):
    return x

  def receive(self, x, mesh_axis, source_pcoord):
    """Processor i receives the slice of processor source_pcoord[i] along
    mesh_axis, zeros where that is None
    (mesh_tensorflow/placement_mesh_impl.py:262-289)."""
    (source,) = source_pcoord
    if source is None:
      return self.slicewise(torch.zeros_like, x)
    return x

  def import_tf_tensor(self, x, tf_x):
    t = torch.as_tensor(tf_x).to(device=self._device, dtype=x.dtype)
    return self.LaidOutTensor([t.contiguous()])

  def export_to_tf_tensor(self, x, laid_out_x):
    return laid_out_x.to_laid_out_tensor().tensor_list[0]

  def random(self, shape, tf_fn, kwargs):
    """tf_fn(sizes, **kwargs) evaluated on the device
    (mesh_tensorflow/placement_mesh_impl.py:307-325)."""
    sizes = self.slice_shape(shape)
    return self.LaidOutTensor([tf_fn(sizes, device=self._device, **kwargs)])
