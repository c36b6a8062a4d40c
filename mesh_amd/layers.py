"""Weight creation for dense layers, as the Mixture-of-Experts layers use it.

Mirrors the part of mesh_tensorflow/layers.py the MoE path touches:
get_dense_kernel_weights (layers.py:211-253: variable `<name>/kernel` of shape
expert_dims + reduced_dims + new_dims) and VarianceScalingInitializer
(layers.py:310-369: truncated normal with stddev sqrt(scale / fan_in)).
The matmul itself is not here: the MoE operations consume the variables
directly.
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
