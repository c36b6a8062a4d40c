"""Dense layers as the Mixture-of-Experts layers and the transformer block
around them use them.

Mirrors the part of mesh_tensorflow/layers.py those paths touch:
get_dense_kernel_weights (layers.py:211-253: variable `<name>/kernel` of shape
expert_dims + reduced_dims + new_dims), VarianceScalingInitializer
(layers.py:310-369: truncated normal with stddev sqrt(scale / fan_in)), and
dense / dense_product without bias (layers.py:112-160, :256-295).  The MoE
operations consume their variables directly.
"""

import torch

from mesh_amd import ops as mtf


class DenseInitializer(object):
  """Initializer that is told (reduced_dims, new_dims) first."""

  def __call__(self, reduced_dims, new_dims):
    raise NotImplementedError("not implemented")


def truncated_normal_initializer(stddev=1.0, seed=None):
  """Normal(0, stddev) redrawn outside two standard deviations, like
  tf.truncated_normal_initializer.  Returns f(sizes, dtype, device)."""
  def init(sizes, dtype, device):
    gen = None
    if seed is not None:
      gen = torch.Generator(device=device)
      gen.manual_seed(seed)
    t = torch.empty(sizes, dtype=torch.float32, device=device)
    torch.nn.init.trunc_normal_(t, mean=0.0, std=stddev, a=-2 * stddev,
                                b=2 * stddev, generator=gen)
    return t.to(dtype)
  return init


def random_normal_initializer(stddev=1.0, seed=None):
  """Normal(0, stddev), like tf.random_normal_initializer.  Returns
  f(sizes, dtype, device)."""
  def init(sizes, dtype, device):
    gen = None
    if seed is not None:
      gen = torch.Generator(device=device)
      gen.manual_seed(seed)
    t = torch.empty(sizes, dtype=torch.float32, device=device)
    t.normal_(0.0, stddev, generator=gen)
    return t.to(dtype)
  return init


def ones_initializer():
  """tf.ones_initializer.  Returns f(sizes, dtype, device)."""
  return lambda sizes, dtype, device: torch.ones(sizes, dtype=dtype,
                                                 device=device)


def random_uniform_initializer(minval, maxval, seed=None):
  def init(sizes, dtype, device):
    gen = None
    if seed is not None:
      gen = torch.Generator(device=device)
      gen.manual_seed(seed)
    t = torch.rand(sizes, dtype=torch.float32, device=device, generator=gen)
    return (t * (maxval - minval) + minval).to(dtype)
  return init


class VarianceScalingInitializer(DenseInitializer):
  """stddev = sqrt(scale / n) with n = fan_in, fan_out or their average."""

  def __init__(self, scale=1.0, mode="fan_in", distribution="normal"):
    self.scale = scale
    self.mode = mode.lower()
    self.distribution = distribution.lower()

  def __call__(self, reduced_dims, new_dims):
    fan_in = mtf.list_product(d.size for d in reduced_dims)
    fan_out = mtf.list_product(d.size for d in new_dims)
    scale = self.scale
    if self.mode == "fan_in":
      scale /= max(1., fan_in)
    elif self.mode == "fan_out":
      scale /= max(1., fan_out)
    elif self.mode == "fan_avg":
      scale /= max(1., float(fan_in + fan_out) / 2)
    else:
      raise ValueError(
          "Invalid `mode` argument: "
          "expected on of {\"fan_in\", \"fan_out\", \"fan_avg\"} "
          "but got %s" % (self.mode,))
    stddev = scale ** 0.5
    if self.distribution == "normal":
      return truncated_normal_initializer(stddev=stddev)
    elif self.distribution == "uniform":
      limit = stddev * 3. ** 0.5
      return random_uniform_initializer(minval=-limit, maxval=limit)
    raise ValueError("Invalid `distribution` argument: "
                     "expected one of {\"normal\", \"uniform\"} "
                     "but got %s" % (self.distribution,))


def get_dense_kernel_weights(x, new_dims, reduced_dims, expert_dims,
                             kernel_initializer, name=None,
                             variable_dtype=None, master_dtype=mtf.float32,
                             slice_dtype=mtf.float32):
  """Creates the variable `<name>/kernel` with shape
  expert_dims + reduced_dims + new_dims and returns its Tensor (in the
  activation dtype)."""
  if variable_dtype is None:
    variable_dtype = mtf.VariableDType(master_dtype, slice_dtype, x.dtype)
  w_shape = mtf.Shape(list(expert_dims) + list(reduced_dims) + list(new_dims))
  with mtf.variable_scope(name or "dense"):
    if kernel_initializer is None:
      kernel_initializer = VarianceScalingInitializer()
    if isinstance(kernel_initializer, DenseInitializer):
      kernel_initializer = kernel_initializer(reduced_dims, new_dims)
    return mtf.get_variable(x.mesh, "kernel", w_shape,
                            initializer=kernel_initializer,
                            dtype=variable_dtype)


class DenseOperation(mtf.Operation):
  """y = activation(x . kernel) over the last dim of x: the einsum (+ relu) of
  mtf.layers.dense without bias (mesh_tensorflow/layers.py:112-160) as one
  operation on the matrix cores.  The kernel is read from the variable's
  K-contiguous packed copy."""

  def __init__(self, x, kernel, new_dims, activation, name=None):
    super(DenseOperation, self).__init__([x, kernel], name=name or "dense")
    self._activation = activation
    shape = mtf.Shape(x.shape.dims[:-1] + list(new_dims))
    self._outputs = [mtf.Tensor(self, shape, x.dtype)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    x, kernel = self.inputs
    mesh_impl = lowering.mesh_impl(self)
    packed = lowering.variables[kernel.operation].packed(x.dtype)
    sizes = self.outputs[0].shape.to_integer_list
    act = self._activation

    def fn(xs):
      return moe_hip.dense(xs.contiguous(), packed, act).reshape(sizes)
    lowering.set_tensor_lowering(
        self.outputs[0], mesh_impl.slicewise(fn, lowering.tensors[x]))

  def gradient(self, grad_ys):
    return list(DenseGradOperation(self, grad_ys[0]).outputs)


class DenseGradOperation(mtf.Operation):
  """(dx, dkernel) of a DenseOperation: what mtf.gradients derives from the
  einsum (mesh_tensorflow/ops.py:2846-2854) and the relu of layers.dense, as
  dpre = dy * (y > 0), dx = dpre . kernel^T, dkernel = x^T . dpre on the
  grouped GEMM with one group."""

  def __init__(self, forward, dy, name=None):
    x, kernel = forward.inputs
    super(DenseGradOperation, self).__init__(
        [dy, x, kernel, forward.outputs[0]], name=name or "dense_grad")
    self._relu = forward._activation == "relu"   # pylint: disable=protected-access
    # When x = relu(dense(...)) feeds nothing but `forward` and nobody asked
    # for d/dx itself, the only reader of dx is the producer's backward, whose
    # first step is the ReLU mask: dx then leaves this operation already
    # multiplied by (x > 0) -- the mask applied on the stores of the GEMM, so
    # dx is d/d(pre-activation) -- and the producer's backward skips its own
    # pass over it (_dy_is_masked below).  Decided here, at gradient time,
    # when every consumer of x is known.
    producer_x = x.operation
    consumers = [op for op in x.graph.operations
                 if x in op.inputs and not isinstance(op, DenseGradOperation)]
    self._masks_dx = (
        isinstance(producer_x, DenseOperation)
        and producer_x._activation == "relu"      # pylint: disable=protected-access
        and x is producer_x.outputs[0]
        and consumers == [forward]
        and not mtf.gradient_is_returned(x))
    # dy already carries this layer's ReLU mask when it is the input gradient
    # of the one operation that consumes the output and that operation masks
    producer = dy.operation
    self._dy_is_masked = (
        self._relu and isinstance(producer, DenseGradOperation)
        and producer._masks_dx and dy is producer.outputs[0]
        and producer.inputs[1] is forward.outputs[0])
    if forward._activation not in (None, "relu"):  # pylint: disable=protected-access
      raise NotImplementedError("gradient of dense with activation %r"
                                % (forward._activation,))  # pylint: disable=protected-access
    self._outputs = [mtf.Tensor(self, x.shape, x.dtype, index=0),
                     mtf.Tensor(self, kernel.shape, kernel.dtype, index=1)]

  def lower(self, lowering):
    from mesh_amd import moe_hip
    mesh_impl = lowering.mesh_impl(self)
    relu = self._relu and not self._dy_is_masked
    masks_dx = self._masks_dx
    k = self.inputs[1].shape.dims[-1].size
    kernel_sizes = self.inputs[2].shape.to_integer_list

    def fn(dy, x, w, y):
      w2 = w.to(x.dtype).reshape(k, -1)
      dx, dw = moe_hip.dense_backward(x.contiguous(), w2, dy.contiguous(),
                                      y if relu else None,
                                      dx_relu_mask=masks_dx)
      return dx, dw.reshape(kernel_sizes).to(w.dtype)
    dx, dw = mesh_impl.slicewise(
        fn, *[lowering.tensors[t] for t in self.inputs])
    lowering.set_tensor_lowering(self.outputs[0], dx)
    lowering.set_tensor_lowering(self.outputs[1], dw)


def _activation_name(activation):
  if activation is None or activation == "linear":
    return None
  name = activation if isinstance(activation, str) else getattr(
      activation, "__name__", None)
  if name != "relu":
    raise NotImplementedError("dense activation %r is not implemented"
                              % (activation,))
  return name


def dense(x, new_dims, reduced_dims=None, expert_dims=None, use_bias=True,
          activation=None, master_dtype=mtf.float32, slice_dtype=mtf.float32,
          variable_dtype=None, kernel_initializer=None, kernel_weights=None,
          name=None):
  """mtf.layers.dense (mesh_tensorflow/layers.py:112-160) for the case the
  transformer layers use: no bias, no expert dims, the reduced dims being the
  trailing dims of x; activation None / "linear" / relu.  The variable is
  `<name>/kernel` with shape reduced_dims + new_dims."""
  if isinstance(new_dims, mtf.Dimension) or not isinstance(new_dims,
                                                           (list, tuple)):
    new_dims = [new_dims]
  new_dims = [mtf.convert_to_dimension(d) for d in new_dims]
  if reduced_dims is None:
    reduced_dims = x.shape.dims[-1:]
  reduced_dims = list(reduced_dims)
  if use_bias:
    raise NotImplementedError("dense with a bias is not implemented")
  if expert_dims:
    raise NotImplementedError("dense with expert (ensemble) dims is not "
                              "implemented; the MoE layers have their own op")
  if kernel_weights is not None:
    raise NotImplementedError("dense with external kernel_weights")
  if len(reduced_dims) != 1 or len(new_dims) != 1:
    raise NotImplementedError("dense over several reduced or new dims")
  if x.shape.dims[-1] != reduced_dims[0]:
    raise NotImplementedError("the reduced dim must be the last dim of x")
  act = _activation_name(activation)
  w = get_dense_kernel_weights(x, new_dims, reduced_dims, [],
                               kernel_initializer, name, variable_dtype,
                               master_dtype, slice_dtype)
  return DenseOperation(x, w, new_dims, act, name=name).outputs[0]


def dense_product(x, reduced_dims, new_dims, activation_functions=None,
                  name="dense_product", **kwargs):
  """mtf.layers.dense_product (mesh_tensorflow/layers.py:256-295) with one
  factor; gated (list) activations are not implemented."""
  if isinstance(activation_functions, list):
    if len(activation_functions) != 1:
      raise NotImplementedError("gated (list) activations are not implemented")
    activation_functions = activation_functions[0]
  return dense(x, new_dims=new_dims, reduced_dims=reduced_dims,
               activation=activation_functions, name=name, **kwargs)
