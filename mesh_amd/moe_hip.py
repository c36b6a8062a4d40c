"""ctypes binding of libmesh_moe_hip.so (declared in include/mesh_moe.h).

The functions here take torch tensors that live on the GPU, check shapes and
dtypes on the host (a kernel launched on mismatched shapes faults the device),
and pass raw device pointers plus the current HIP stream through the C ABI.
torch is used for device memory and streams only.

There is no CPU fallback: if the shared library has not been built, loading
raises, and so does every call.
"""

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmesh_moe_hip.so")

F32 = 0
BF16 = 1
POLICIES = {"all": 0, "none": 1, "threshold": 2, "random": 3}
ACTIVATIONS = {None: 0, "linear": 0, "relu": 1, "gelu": 2, "sigmoid": 3,
               "tanh": 4, "swish": 5}
ABI_VERSION = 34

_vp = ctypes.c_void_p
_SIGNATURES = {
    "mesh_moe_abi_version": (ctypes.c_int, []),
    "mesh_moe_last_error": (ctypes.c_char_p, []),
    "mesh_moe_crc32c": (ctypes.c_uint32, [
        ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t]),
    "mesh_moe_router_logits": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_gating_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_top2_gating": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_int,
        ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t,
        _vp]),
    "mesh_moe_top2_gating_static_scratch": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_int,
        ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mesh_moe_router_top2_gating": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_double, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp, _vp,
        _vp, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_switch_gating": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_double,
        ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t,
        _vp]),
    "mesh_moe_router_switch_gating": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_double, ctypes.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
        ctypes.c_size_t, _vp]),
    "mesh_moe_ntlb_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_ntlb_gating": (ctypes.c_int, [
        _vp, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp, _vp,
        _vp, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_router_summaries_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_router_summaries": (ctypes.c_int, [
        _vp, ctypes.c_int, _vp, ctypes.c_int, _vp, _vp, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, _vp, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_dispatch": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_pack_weights": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, _vp]),
    "mesh_moe_expert_ffn": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_dispatched_expert_ffn_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_dispatched_expert_ffn": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_compact_expert_ffn_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int]),
    "mesh_moe_compact_expert_ffn": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
        ctypes.c_float, _vp, _vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp]),
    "mesh_moe_combine_compact": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_dispatch_compact": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_combine_backward_compact": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp]),
    "mesh_moe_compact_expert_ffn_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int]),
    "mesh_moe_compact_expert_ffn_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp,
        ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_dispatch_backward_compact": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, _vp]),
    "mesh_moe_expert_linear": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_combine": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_combine_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp]),
    "mesh_moe_expert_ffn_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int]),
    "mesh_moe_hidden_product": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_float, _vp, ctypes.c_int64, ctypes.c_int, _vp]),
    "mesh_moe_expert_ffn_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp,
        ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_expert_linear_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_expert_linear_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_rms_norm_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int64, ctypes.c_int]),
    "mesh_moe_rms_norm_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_double,
        ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_softmax_backward": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_attention_weights_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_attention_weights": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, _vp,
        ctypes.c_size_t, _vp]),
    "mesh_moe_relative_bias_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_broadcast_dropout": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_float, _vp, _vp, ctypes.c_int64, ctypes.c_int64,
        ctypes.c_int64, ctypes.c_int, _vp]),
    "mesh_moe_activation": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_activation_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_slot_combine_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_slot_dispatch_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_expert_choice_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_expert_choice_backward": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, _vp, _vp, _vp, ctypes.c_double, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_gating_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int]),
    "mesh_moe_gating_backward": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp,
        ctypes.c_double,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_int, _vp, _vp,
        ctypes.c_size_t, _vp]),
    "mesh_moe_router_backward_weights_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_router_backward_weights": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, _vp]),
    "mesh_moe_dispatch_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _vp]),
    "mesh_moe_expert_choice_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mesh_moe_expert_choice_gating": (ctypes.c_int, [
        _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp, _vp,
        ctypes.c_size_t, _vp]),
    "mesh_moe_slot_dispatch": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_slot_combine": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp]),
    "mesh_moe_rms_norm": (ctypes.c_int, [
        _vp, _vp, _vp, ctypes.c_int64, ctypes.c_int, ctypes.c_double,
        ctypes.c_int, _vp]),
    "mesh_moe_self_attention_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int]),
    "mesh_moe_self_attention": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, ctypes.c_int, _vp,
        ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_self_attention_backward_workspace_bytes": (ctypes.c_size_t, [
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_int]),
    "mesh_moe_self_attention_backward": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, ctypes.c_int,
        _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "mesh_moe_attention_decode": (ctypes.c_int, [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _vp, _vp, ctypes.c_int, ctypes.c_int, _vp]),
}
EXPORTS = sorted(_SIGNATURES)

_lib = None


class MoeHipError(RuntimeError):
  """A call into libmesh_moe_hip.so was rejected."""


def load_library(path=None):
  """Loads the shared library (once) and declares every entry point."""
  global _lib
  if _lib is not None and path is None:
    return _lib
  path = path or LIB_PATH
  if not os.path.exists(path):
    raise MoeHipError(
        "%s not found: build it with `python -m mesh_amd.csrc.build` "
        "(there is no CPU fallback)" % path)
  lib = ctypes.CDLL(path)
  for name, (restype, argtypes) in _SIGNATURES.items():
    fn = getattr(lib, name)  # AttributeError if a symbol is missing
    fn.restype = restype
    fn.argtypes = argtypes
  version = lib.mesh_moe_abi_version()
  if version != ABI_VERSION:
    raise MoeHipError("ABI version %d, expected %d" % (version, ABI_VERSION))
  _lib = lib
  return lib


def _check(rc, what):
  if rc != 0:
    msg = load_library().mesh_moe_last_error().decode("utf-8", "replace")
    raise MoeHipError("%s failed (%d): %s" % (what, rc, msg))


def dtype_code(dtype):
  if dtype == torch.float32:
    return F32
  if dtype == torch.bfloat16:
    return BF16
  raise MoeHipError("unsupported dtype %s (float32 and bfloat16 only)" % dtype)


def _dev(t, name, dtype=None, shape=None):
  if not isinstance(t, torch.Tensor) or not t.is_cuda:
    raise MoeHipError("%s must be a GPU tensor" % name)
  if not t.is_contiguous():
    raise MoeHipError("%s must be contiguous" % name)
  if dtype is not None and t.dtype != dtype:
    raise MoeHipError("%s: dtype %s, expected %s" % (name, t.dtype, dtype))
  if shape is not None and tuple(t.shape) != tuple(shape):
    raise MoeHipError("%s: shape %s, expected %s"
                      % (name, tuple(t.shape), tuple(shape)))
  return t.data_ptr()


def _stream():
  return torch.cuda.current_stream().cuda_stream


class StageTimer(object):
  """Optional per-stage HIP-event timing of the calls below.

  While a StageTimer is installed (`with StageTimer() as t:`), every stage
  records a start and an end event on the stream it launches on; `totals()`
  synchronises and returns {stage: (calls, milliseconds)}.  The last Routing
  produced is kept in `routing` so that a benchmark can count kept slots;
  `compacted` counts the expert feed-forward calls that ran on compacted
  rows (only the occupied slots multiplied).  With keep_calls=True the last
  library call of the router and combine stages is kept in `calls` (function,
  arguments and the tensors behind the pointers) for back_to_back_ms().
  """

  def __init__(self, keep_calls=False):
    self.events = []
    self.routing = []
    self.compacted = 0
    self.keep_calls = keep_calls
    self.calls = {}

  def __enter__(self):
    global _timer
    self._previous = _timer
    _timer = self
    return self

  def __exit__(self, *exc):
    global _timer
    _timer = self._previous
    return False

  def totals(self):
    torch.cuda.synchronize()
    out = {}
    for name, start, end in self.events:
      calls, ms = out.get(name, (0, 0.0))
      out[name] = (calls + 1, ms + start.elapsed_time(end))
    return out


_timer = None


class _stage(object):
  """Context manager bracketing one stage with events if a timer is set."""

  def __init__(self, name):
    self.name = name

  def __enter__(self):
    if _timer is not None:
      self.start = torch.cuda.Event(enable_timing=True)
      self.start.record()
    return self

  def __exit__(self, *exc):
    if _timer is not None and exc[0] is None:
      end = torch.cuda.Event(enable_timing=True)
      end.record()
      _timer.events.append((self.name, self.start, end))
    return False

  def call(self, keep, fn, *args):
    """Makes the stage's library call fn(*args); a timer with keep_calls
    remembers it together with `keep`, the tensors whose addresses args
    holds."""
    if _timer is not None and _timer.keep_calls:
      _timer.calls[self.name] = (fn, args, keep)
    return fn(*args)


def back_to_back_ms(call, reps=50, warmup=3):
  """Average duration in ms of `reps` launches of a call kept by
  StageTimer(keep_calls=True), issued back to back between ONE pair of events
  on the current stream: the stage's launches without the cost of an event
  pair around each of them.  The call rewrites its own outputs with the same
  values."""
  fn, args, _ = call
  for _ in range(warmup):
    _check(fn(*args), "back_to_back warm-up")
  start = torch.cuda.Event(enable_timing=True)
  end = torch.cuda.Event(enable_timing=True)
  start.record()
  for _ in range(reps):
    rc = fn(*args)
    if rc != 0:
      _check(rc, "back_to_back")
  end.record()
  end.synchronize()
  return start.elapsed_time(end) / reps


def router_logits(x, w, bias=None, out=None, w_packed=None):
  """x [B, T, M] or [T, M]; w [B, M, E] or [M, E] -> float32 logits [.., T, E].
  w_packed, if given, is pack_weights(w): [B, E, M] (or [E, M])."""
  lib = load_library()
  squeeze = x.dim() == 2
  if squeeze:
    x, w = x.unsqueeze(0), w.unsqueeze(0)
    if w_packed is not None and w_packed.dim() == 2:
      w_packed = w_packed.unsqueeze(0)
  b, t, m = x.shape
  e = w.shape[-1]
  code = dtype_code(x.dtype)
  xp = _dev(x, "x")
  wp = _dev(w, "w", x.dtype, (b, m, e))
  if out is None:
    out = torch.empty((b, t, e), dtype=torch.float32, device=x.device)
  op = _dev(out, "logits", torch.float32, (b, t, e))
  bp = None if bias is None else _dev(bias, "bias", torch.float32, (e,))
  pp = None if w_packed is None else _dev(w_packed, "w_packed", x.dtype,
                                          (b, e, m))
  with _stage("router_logits"):
    _check(lib.mesh_moe_router_logits(xp, wp, pp, bp, op, b, t, m, e, code,
                                      _stream()), "router_logits")
  return out[0] if squeeze else out


class Routing(object):
  """Per-token routing record written by top2_gating."""

  def __init__(self, idx, pos, gate, kept, fill, loss, capacity, num_experts):
    self.idx, self.pos, self.gate, self.kept = idx, pos, gate, kept
    self.fill, self.loss = fill, loss
    self.capacity, self.num_experts = capacity, num_experts


def top2_gating(logits, capacity, importance=None, policy="all",
                threshold=0.2, use_second_place_loss=False,
                num_microbatches=None, second_uniform=None,
                importance_from_slot_gate=False):
  """logits float32 [G, S, E] -> Routing (all tensors on the GPU)."""
  lib = load_library()
  if policy not in POLICIES:
    raise ValueError("Unknown policy %s" % policy)
  g, s, e = logits.shape
  lp = _dev(logits, "logits", torch.float32)
  dev = logits.device
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  up = None
  if second_uniform is not None:
    up = _dev(second_uniform, "second_uniform", torch.float32, (g, s))
  idx = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  pos = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  gate = torch.empty((g, s, 2), dtype=torch.float32, device=dev)
  kept = torch.empty((g, s, 2), dtype=torch.uint8, device=dev)
  fill = torch.empty((g, e), dtype=torch.int32, device=dev)
  loss = torch.empty((1,), dtype=torch.float32, device=dev)
  ws_bytes = lib.mesh_moe_gating_workspace_bytes(g, s, e)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("top2_gating"):
    _check(lib.mesh_moe_top2_gating(
        lp, ip, icode, int(bool(importance_from_slot_gate)), up, g, s, e,
        int(capacity), POLICIES[policy],
        float(threshold), int(bool(use_second_place_loss)),
        int(num_microbatches or 1), idx.data_ptr(), pos.data_ptr(),
        gate.data_ptr(), kept.data_ptr(), fill.data_ptr(), loss.data_ptr(),
        ws.data_ptr(), ws_bytes, _stream()), "top2_gating")
  r = Routing(idx, pos, gate, kept, fill, loss, int(capacity), e)
  if _timer is not None:
    _timer.routing.append(r)
  return r


STATIC_SCRATCH_BYTES = 4 << 20


def top2_gating_static_scratch(logits, capacity, out, importance=None,
                               policy="all", threshold=0.2,
                               use_second_place_loss=False,
                               num_microbatches=None, second_uniform=None,
                               importance_from_slot_gate=False):
  """top2_gating into the caller's Routing `out`, on the library's built-in
  scratch array: neither this function nor the call behind it allocates.
  Calls that overlap on one GPU race for that array."""
  lib = load_library()
  if policy not in POLICIES:
    raise ValueError("Unknown policy %s" % policy)
  g, s, e = logits.shape
  lp = _dev(logits, "logits", torch.float32)
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  up = None
  if second_uniform is not None:
    up = _dev(second_uniform, "second_uniform", torch.float32, (g, s))
  ptrs = [_dev(out.idx, "idx", torch.int32, (g, s, 2)),
          _dev(out.pos, "pos", torch.int32, (g, s, 2)),
          _dev(out.gate, "gate", torch.float32, (g, s, 2)),
          _dev(out.kept, "kept", torch.uint8, (g, s, 2)),
          _dev(out.fill, "fill", torch.int32, (g, e)),
          _dev(out.loss, "loss", torch.float32, (1,))]
  with _stage("top2_gating"):
    _check(lib.mesh_moe_top2_gating_static_scratch(
        lp, ip, icode, int(bool(importance_from_slot_gate)), up, g, s, e,
        int(capacity), POLICIES[policy], float(threshold),
        int(bool(use_second_place_loss)), int(num_microbatches or 1),
        *ptrs, _stream()), "top2_gating_static_scratch")
  out.capacity, out.num_experts = int(capacity), e
  return out


def fused_gating_supported(x, num_experts, group_size):
  """True if mesh_moe_router_top2_gating has a kernel for this case."""
  return (x.dtype == torch.bfloat16 and x.shape[-1] % 64 == 0 and
          num_experts % 4 == 0 and num_experts <= 128 and group_size % 128 == 0)


def router_top2_gating(x, w_packed, group_size, capacity, importance=None,
                       policy="all", threshold=0.2,
                       use_second_place_loss=False, num_microbatches=None,
                       second_uniform=None, importance_from_slot_gate=False,
                       bias=None, want_logits=False):
  """Router projection + top-2 gating in one launch sequence.

  x [B, T, M] bf16 with w_packed [B, E, M] (one router per leading index), the
  B*T tokens forming groups of `group_size`.  Returns Routing over
  [G = B*T/group_size, group_size] (and the logits if want_logits)."""
  lib = load_library()
  if policy not in POLICIES:
    raise ValueError("Unknown policy %s" % policy)
  b, t, m = x.shape
  e = w_packed.shape[1]
  s = int(group_size)
  if (b * t) % s or t % s:
    raise MoeHipError("tokens per router (%d) must be whole groups of %d"
                      % (t, s))
  g = b * t // s
  dev = x.device
  xp = _dev(x, "x", torch.bfloat16)
  wp = _dev(w_packed, "w_packed", torch.bfloat16, (b, e, m))
  bp = None if bias is None else _dev(bias, "bias", torch.float32, (e,))
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  up = None
  if second_uniform is not None:
    up = _dev(second_uniform, "second_uniform", torch.float32, (g, s))
  logits = None
  if want_logits:
    logits = torch.empty((g, s, e), dtype=torch.float32, device=dev)
  idx = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  pos = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  gate = torch.empty((g, s, 2), dtype=torch.float32, device=dev)
  kept = torch.empty((g, s, 2), dtype=torch.uint8, device=dev)
  fill = torch.empty((g, e), dtype=torch.int32, device=dev)
  loss = torch.empty((1,), dtype=torch.float32, device=dev)
  ws_bytes = lib.mesh_moe_gating_workspace_bytes(g, s, e)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("router_top2_gating") as st:
    _check(st.call(
        (x, w_packed, bias, importance, second_uniform, logits, idx, pos, gate,
         kept, fill, loss, ws), lib.mesh_moe_router_top2_gating,
        xp, wp, bp, None if logits is None else logits.data_ptr(), b, t, m,
        BF16, ip, icode, int(bool(importance_from_slot_gate)), up, g, s, e,
        int(capacity), POLICIES[policy], float(threshold),
        int(bool(use_second_place_loss)), int(num_microbatches or 1),
        idx.data_ptr(), pos.data_ptr(), gate.data_ptr(), kept.data_ptr(),
        fill.data_ptr(), loss.data_ptr(), ws.data_ptr(), ws_bytes, _stream()),
        "router_top2_gating")
  r = Routing(idx, pos, gate, kept, fill, loss, int(capacity), e)
  if _timer is not None:
    _timer.routing.append(r)
  return (r, logits) if want_logits else r


def _routing_buffers(lib, g, s, e, dev):
  idx = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  pos = torch.empty((g, s, 2), dtype=torch.int32, device=dev)
  gate = torch.empty((g, s, 2), dtype=torch.float32, device=dev)
  kept = torch.empty((g, s, 2), dtype=torch.uint8, device=dev)
  fill = torch.empty((g, e), dtype=torch.int32, device=dev)
  loss = torch.empty((1,), dtype=torch.float32, device=dev)
  ws_bytes = lib.mesh_moe_gating_workspace_bytes(g, s, e)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  return idx, pos, gate, kept, fill, loss, ws, ws_bytes


def switch_gating(logits, capacity, importance=None, z_loss=None,
                  num_microbatches=None, slots_by_gate=False,
                  choice_logits=None):
  """logits float32 [G, S, E] -> Routing for switch (top-1) gating.

  choice_logits float32 [G, S, E]: when given, the expert of a token is the
  first arg-max of its row there (policy "sample", transformer/moe.py:1213-1216)
  and the gate is the softmax probability of that expert.

  z_loss: coefficient of the router z-loss, or None to leave it out (the
  caller passes it only when training, transformer/moe.py:1253).
  slots_by_gate: an expert keeps its choosers with the largest gate instead of
  the earliest ones (_switch_max_gating, transformer/moe.py:1033-1039)."""
  lib = load_library()
  g, s, e = logits.shape
  lp = _dev(logits, "logits", torch.float32)
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  idx, pos, gate, kept, fill, loss, ws, ws_bytes = _routing_buffers(
      lib, g, s, e, logits.device)
  with _stage("switch_gating"):
    cp = None if choice_logits is None else _dev(
        choice_logits, "choice_logits", torch.float32, (g, s, e))
    _check(lib.mesh_moe_switch_gating(
        lp, cp, ip, icode, g, s, e, int(capacity), int(bool(slots_by_gate)),
        int(z_loss is not None), float(z_loss or 0.0),
        int(num_microbatches or 1), idx.data_ptr(),
        pos.data_ptr(), gate.data_ptr(), kept.data_ptr(), fill.data_ptr(),
        loss.data_ptr(), ws.data_ptr(), ws_bytes, _stream()), "switch_gating")
  r = Routing(idx, pos, gate, kept, fill, loss, int(capacity), e)
  if _timer is not None:
    _timer.routing.append(r)
  return r


def ntlb_gating(logits, capacity, top_k, importance=None,
                num_microbatches=None, softmax_dtype=torch.float32):
  """logits float32 [G, S, E] -> Routing for "no token left behind" gating
  (_ntlb_gating, transformer/moe.py:804-940): top_k candidates per token, one
  pass per candidate rank, each token routed at most once.  softmax_dtype:
  the activation dtype -- this router runs its projection's result and its
  softmax in it (moe.py:825-836); with torch.bfloat16 the logits are rounded
  and every softmax op rounds to bfloat16."""
  lib = load_library()
  g, s, e = logits.shape
  lp = _dev(logits, "logits", torch.float32)
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  idx, pos, gate, kept, fill, loss, _, _ = _routing_buffers(
      lib, g, s, e, logits.device)
  ws_bytes = lib.mesh_moe_ntlb_workspace_bytes(g, s, e, int(top_k))
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8,
                   device=logits.device)
  with _stage("ntlb_gating"):
    _check(lib.mesh_moe_ntlb_gating(
        lp, dtype_code(softmax_dtype), ip, icode, g, s, e, int(capacity),
        int(top_k),
        int(num_microbatches or 1), idx.data_ptr(), pos.data_ptr(),
        gate.data_ptr(), kept.data_ptr(), fill.data_ptr(), loss.data_ptr(),
        ws.data_ptr(), ws_bytes, _stream()), "ntlb_gating")
  r = Routing(idx, pos, gate, kept, fill, loss, int(capacity), e)
  if _timer is not None:
    _timer.routing.append(r)
  return r


SUMMARY_ROUTERS = {"switch": 1, "switch_max": 1, "ntlb": 2,
                   "expert_selection": 3}


def router_summaries(logits, router, capacity, importance=None, kept=None,
                     tok_slot=None, top_k=1, num_microbatches=None,
                     softmax_dtype=torch.float32):
  """The values the f1 routers hand to mtf.scalar_summary while training
  (transformer/moe.py:865-880, :981, :1010-1025, :1041-1046, :1149-1165, :1213,
  :1242-1257, :1259-1269, :1285-1289), from the router's float32 logits
  [G, S, E] and its record.  Returns a float32 tensor: [0] mean entropy, [1]
  mean largest probability, [2] fraction routed, [3] z-loss, then per expert
  its share of the routed choices (switch, switch_max, ntlb: E values) or per
  group position E * C * the number of experts that took it (expert selection:
  S values)."""
  lib = load_library()
  g, s, e = logits.shape
  code = SUMMARY_ROUTERS[router]
  lp = _dev(logits, "logits", torch.float32)
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  kp = None if kept is None else _dev(kept, "kept", torch.uint8, (g, s, 2))
  tp = None if tok_slot is None else _dev(tok_slot, "tok_slot", torch.int16,
                                          (g, s, e))
  out = torch.empty((4 + (s if code == 3 else e),), dtype=torch.float32,
                    device=logits.device)
  ws_bytes = lib.mesh_moe_router_summaries_workspace_bytes(g, s, e)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8,
                   device=logits.device)
  with _stage("router_summaries"):
    _check(lib.mesh_moe_router_summaries(
        lp, dtype_code(softmax_dtype), ip, icode, kp, tp, g, s, e,
        int(capacity), code, int(top_k), int(num_microbatches or 1),
        out.data_ptr(), ws.data_ptr(), ws_bytes, _stream()),
           "router_summaries")
  return out


def router_switch_gating(x, w_packed, group_size, capacity, importance=None,
                         z_loss=None, num_microbatches=None, bias=None,
                         want_logits=False, slots_by_gate=False):
  """Router projection + switch gating in one launch sequence; arguments as
  router_top2_gating / switch_gating."""
  lib = load_library()
  b, t, m = x.shape
  e = w_packed.shape[1]
  s = int(group_size)
  if (b * t) % s or t % s:
    raise MoeHipError("tokens per router (%d) must be whole groups of %d"
                      % (t, s))
  g = b * t // s
  dev = x.device
  xp = _dev(x, "x", torch.bfloat16)
  wp = _dev(w_packed, "w_packed", torch.bfloat16, (b, e, m))
  bp = None if bias is None else _dev(bias, "bias", torch.float32, (e,))
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  logits = None
  if want_logits:
    logits = torch.empty((g, s, e), dtype=torch.float32, device=dev)
  idx, pos, gate, kept, fill, loss, ws, ws_bytes = _routing_buffers(
      lib, g, s, e, dev)
  with _stage("router_switch_gating") as st:
    _check(st.call(
        (x, w_packed, bias, importance, logits, idx, pos, gate, kept, fill,
         loss, ws), lib.mesh_moe_router_switch_gating,
        xp, wp, bp, None if logits is None else logits.data_ptr(), b, t, m,
        BF16, ip, icode, g, s, e, int(capacity), int(bool(slots_by_gate)),
        int(z_loss is not None), float(z_loss or 0.0),
        int(num_microbatches or 1), idx.data_ptr(),
        pos.data_ptr(), gate.data_ptr(), kept.data_ptr(), fill.data_ptr(),
        loss.data_ptr(), ws.data_ptr(), ws_bytes, _stream()),
        "router_switch_gating")
  r = Routing(idx, pos, gate, kept, fill, loss, int(capacity), e)
  if _timer is not None:
    _timer.routing.append(r)
  return (r, logits) if want_logits else r


def dispatch(x, r, want_slot_gate=False, out=None, row_offsets=None):
  """x [G, S, M] -> expert_in [E, G, C, M] (and slot_gate [E, G, C]).  With
  row_offsets [E, G] (from compact_expert_ffn) every expert's occupied slots
  go to the front of its rows."""
  lib = load_library()
  g, s, m = x.shape
  e, c = r.num_experts, r.capacity
  code = dtype_code(x.dtype)
  xp = _dev(x, "x")
  if out is None:
    out = torch.empty((e, g, c, m), dtype=x.dtype, device=x.device)
  op = _dev(out, "expert_in", x.dtype, (e, g, c, m))
  if row_offsets is not None:
    if want_slot_gate:
      raise MoeHipError("dispatch: no slot gates with compacted rows")
    ip, pp, gp, kp = _routing_ptrs(r, g, s)
    with _stage("dispatch"):
      _check(lib.mesh_moe_dispatch_compact(
          xp, ip, pp, gp, kp, _dev(r.fill, "fill", torch.int32, (g, e)),
          _dev(row_offsets, "row_offsets", torch.int32, (e, g)), op, g, s, e,
          c, m, code, _stream()), "dispatch_compact")
    return out
  slot_gate = None
  if want_slot_gate:
    slot_gate = torch.empty((e, g, c), dtype=torch.float32, device=x.device)
  with _stage("dispatch"):
    _check(lib.mesh_moe_dispatch(
        xp, _dev(r.idx, "idx", torch.int32, (g, s, 2)),
        _dev(r.pos, "pos", torch.int32, (g, s, 2)),
        _dev(r.gate, "gate", torch.float32, (g, s, 2)),
        _dev(r.kept, "kept", torch.uint8, (g, s, 2)),
        _dev(r.fill, "fill", torch.int32, (g, e)), op,
        None if slot_gate is None else slot_gate.data_ptr(),
        g, s, e, c, m, code, _stream()), "dispatch")
  return (out, slot_gate) if want_slot_gate else out


def pack_weights(w, dtype, out=None):
  """w [E, K, N] (any supported dtype) -> packed [E, N, K] of `dtype`, into
  `out` if given."""
  lib = load_library()
  e, k, n = w.shape
  if out is None:
    out = torch.empty((e, n, k), dtype=dtype, device=w.device)
  _dev(out, "packed", dtype, (e, n, k))
  _check(lib.mesh_moe_pack_weights(
      _dev(w, "w"), out.data_ptr(), e, k, n, dtype_code(w.dtype),
      dtype_code(dtype), _stream()), "pack_weights")
  return out


def expert_ffn(expert_in, wi_packed, wo_packed, activation="relu", h=None,
               y=None):
  """expert_in [E, R, M]; wi_packed [E, H, M]; wo_packed [E, N, H] -> y [E,R,N]."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  e, rows, m = expert_in.shape
  hdim = wi_packed.shape[1]
  n = wo_packed.shape[1]
  dt = expert_in.dtype
  code = dtype_code(dt)
  ip = _dev(expert_in, "expert_in")
  wip = _dev(wi_packed, "wi_packed", dt, (e, hdim, m))
  wop = _dev(wo_packed, "wo_packed", dt, (e, n, hdim))
  if h is None:
    h = torch.empty((e, rows, hdim), dtype=dt, device=expert_in.device)
  if y is None:
    y = torch.empty((e, rows, n), dtype=dt, device=expert_in.device)
  hp = _dev(h, "h", dt, (e, rows, hdim))
  yp = _dev(y, "y", dt, (e, rows, n))
  with _stage("expert_ffn"):
    _check(lib.mesh_moe_expert_ffn(ip, wip, wop, hp, yp, e, rows, m, hdim, n,
                                   ACTIVATIONS[activation], code, _stream()),
           "expert_ffn")
  return y


E_UNSUPPORTED = -2


def dispatched_expert_ffn(x, r, wi_packed, wo_packed, activation="relu",
                          h=None):
  """dispatch + expert_ffn without materialising expert_in: x [G, S, M], the
  Routing r -> y [E, G*C, N], or None where the library has no such kernel for
  the case (the caller then makes the two calls).  h [E, G*C, H], if given,
  receives the hidden tensor."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  g, s, m = x.shape
  e, c = r.num_experts, r.capacity
  hdim, n = wi_packed.shape[1], wo_packed.shape[1]
  dt = x.dtype
  if dt != torch.bfloat16:
    return None
  dev = x.device
  if h is None:
    h = torch.empty((e, g * c, hdim), dtype=dt, device=dev)
  _dev(h, "h", dt, (e, g * c, hdim))
  y = torch.empty((e, g * c, n), dtype=dt, device=dev)
  ws_bytes = lib.mesh_moe_dispatched_expert_ffn_workspace_bytes(g, e, c, m)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("expert_ffn"):
    rc = lib.mesh_moe_dispatched_expert_ffn(
        _dev(x, "x"), _dev(r.idx, "idx", torch.int32, (g, s, 2)),
        r.pos.data_ptr(), r.gate.data_ptr(), r.kept.data_ptr(),
        _dev(wi_packed, "wi_packed", dt, (e, hdim, m)),
        _dev(wo_packed, "wo_packed", dt, (e, n, hdim)), h.data_ptr(),
        y.data_ptr(), ws.data_ptr(), ws_bytes, g, s, e, c, m, hdim, n,
        ACTIVATIONS[activation], dtype_code(dt), _stream())
  if rc == E_UNSUPPORTED:
    return None
  _check(rc, "dispatched_expert_ffn")
  return y


def compact_training_applies(x, r, hidden_size, output_size,
                             activation="relu"):
  """True if a layer's gradient graph can stay on compacted rows: the forward
  call compact_expert_ffn and the compacted gradient calls all take the
  case."""
  lib = load_library()
  g, s, m = x.shape
  e, c = r.num_experts, r.capacity
  return (x.dtype == torch.bfloat16 and activation in ("relu", "linear") and
          lib.mesh_moe_compact_expert_ffn_backward_workspace_bytes(
              g, e, c, m, hidden_size, output_size) > 0)


def compact_expert_ffn(x, r, wi_packed, wo_packed, activation="relu",
                       want_hidden=False, uniform=None, keep_prob=1.0,
                       want_noise=False):
  """dispatch + expert_ffn on compacted rows (only the tiles that hold
  occupied slots are multiplied): x [G, S, M], the Routing r -> (y [E, G*C, N],
  row_offsets [E, G]) for combine(..., row_offsets=...), or None where the
  library has no such kernel for the case.  want_hidden: (y, row_offsets, h)
  with the hidden tensor h [E, G*C, H] in the same row order.  uniform
  [E, G*C, H]: the hidden dropout h *= (uniform < keep_prob) / keep_prob
  between the two products; want_noise appends the noise tensor to the
  result."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  g, s, m = x.shape
  e, c = r.num_experts, r.capacity
  hdim, n = wi_packed.shape[1], wo_packed.shape[1]
  dt = x.dtype
  if dt != torch.bfloat16:
    return None
  dev = x.device
  h = torch.empty((e, g * c, hdim), dtype=dt, device=dev)
  y = torch.empty((e, g * c, n), dtype=dt, device=dev)
  row_offsets = torch.empty((e, g), dtype=torch.int32, device=dev)
  noise = (torch.empty_like(h) if (want_noise and uniform is not None)
           else None)
  ws_bytes = lib.mesh_moe_compact_expert_ffn_workspace_bytes(g, e, c, m, hdim, n)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("expert_ffn"):
    rc = lib.mesh_moe_compact_expert_ffn(
        _dev(x, "x"), _dev(r.idx, "idx", torch.int32, (g, s, 2)),
        r.pos.data_ptr(), r.gate.data_ptr(), r.kept.data_ptr(),
        _dev(r.fill, "fill", torch.int32, (g, e)),
        _dev(wi_packed, "wi_packed", dt, (e, hdim, m)),
        _dev(wo_packed, "wo_packed", dt, (e, n, hdim)), h.data_ptr(),
        y.data_ptr(), row_offsets.data_ptr(),
        _dev(uniform, "uniform", dt, (e, g * c, hdim))
        if uniform is not None else None, float(keep_prob),
        noise.data_ptr() if noise is not None else None,
        ws.data_ptr(), ws_bytes, g, s, e,
        c, m, hdim, n, ACTIVATIONS[activation], dtype_code(dt), _stream())
  if rc == E_UNSUPPORTED:
    return None
  _check(rc, "compact_expert_ffn")
  if _timer is not None:
    _timer.compacted += 1
  res = (y, row_offsets, h) if want_hidden else (y, row_offsets)
  return res + (noise,) if want_noise else res


def expert_linear(a, w_packed, activation="linear", y=None):
  """a [E, R, K]; w_packed [E, N, K] -> y [E, R, N] = act(a . w) per expert."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  e, rows, k = a.shape
  n = w_packed.shape[1]
  dt = a.dtype
  if y is None:
    y = torch.empty((e, rows, n), dtype=dt, device=a.device)
  with _stage("expert_linear"):
    _check(lib.mesh_moe_expert_linear(
        _dev(a, "a"), _dev(w_packed, "w_packed", dt, (e, n, k)),
        _dev(y, "y", dt, (e, rows, n)), e, rows, k, n, ACTIVATIONS[activation],
        dtype_code(dt), _stream()), "expert_linear")
  return y


def combine(y, r, group_size, out=None, row_offsets=None):
  """y [E, G, C, N] -> out [G, S, N].  With row_offsets [E, G] (from
  compact_expert_ffn) y holds every expert's occupied slots first."""
  lib = load_library()
  e, g, c, n = y.shape
  s = group_size
  code = dtype_code(y.dtype)
  yp = _dev(y, "y")
  if (e, c) != (r.num_experts, r.capacity):
    raise MoeHipError("combine: y is [E=%d, C=%d], routing has E=%d, C=%d"
                      % (e, c, r.num_experts, r.capacity))
  if out is None:
    out = torch.empty((g, s, n), dtype=y.dtype, device=y.device)
  op = _dev(out, "out", y.dtype, (g, s, n))
  if row_offsets is not None:
    with _stage("combine") as st:
      _check(st.call(
          (y, r, row_offsets, out), lib.mesh_moe_combine_compact,
          yp, _dev(r.idx, "idx", torch.int32, (g, s, 2)),
          _dev(r.pos, "pos", torch.int32, (g, s, 2)),
          _dev(r.gate, "gate", torch.float32, (g, s, 2)),
          _dev(r.kept, "kept", torch.uint8, (g, s, 2)),
          _dev(row_offsets, "row_offsets", torch.int32, (e, g)), op, g, s, e, c,
          n, code, _stream()), "combine_compact")
    return out
  with _stage("combine") as st:
    _check(st.call(
        (y, r, out), lib.mesh_moe_combine,
        yp, _dev(r.idx, "idx", torch.int32, (g, s, 2)),
        _dev(r.pos, "pos", torch.int32, (g, s, 2)),
        _dev(r.gate, "gate", torch.float32, (g, s, 2)),
        _dev(r.kept, "kept", torch.uint8, (g, s, 2)), op, g, s, e, c, n, code,
        _stream()), "combine")
  return out


# ----------------------------------------------------------------------------
# backward
# ----------------------------------------------------------------------------
def _routing_ptrs(r, g, s):
  return (_dev(r.idx, "idx", torch.int32, (g, s, 2)),
          _dev(r.pos, "pos", torch.int32, (g, s, 2)),
          _dev(r.gate, "gate", torch.float32, (g, s, 2)),
          _dev(r.kept, "kept", torch.uint8, (g, s, 2)))


def combine_backward(dout, y, r, row_offsets=None):
  """dout [G, S, N], y [E, G, C, N] -> (dy [E, G, C, N], dgate [G, S, 2]).
  With row_offsets [E, G], y and dy hold every expert's occupied slots
  first."""
  lib = load_library()
  g, s, n = dout.shape
  e, _, c, _ = y.shape
  dt = y.dtype
  dy = torch.empty_like(y)
  dgate = torch.empty((g, s, 2), dtype=torch.float32, device=y.device)
  ip, pp, gp, kp = _routing_ptrs(r, g, s)
  if row_offsets is not None:
    with _stage("combine_backward"):
      _check(lib.mesh_moe_combine_backward_compact(
          _dev(dout, "dout", dt, (g, s, n)), _dev(y, "y", dt, (e, g, c, n)),
          ip, pp, gp, kp, _dev(r.fill, "fill", torch.int32, (g, e)),
          _dev(row_offsets, "row_offsets", torch.int32, (e, g)),
          dy.data_ptr(), dgate.data_ptr(), g, s, e, c, n, dtype_code(dt),
          _stream()), "combine_backward_compact")
    return dy, dgate
  with _stage("combine_backward"):
    _check(lib.mesh_moe_combine_backward(
        _dev(dout, "dout", dt, (g, s, n)), _dev(y, "y", dt, (e, g, c, n)),
        ip, pp, gp, kp, _dev(r.fill, "fill", torch.int32, (g, e)),
        dy.data_ptr(), dgate.data_ptr(), g, s, e, c, n, dtype_code(dt),
        _stream()), "combine_backward")
  return dy, dgate


def hidden_product(h, factor=None, uniform=None, keep_prob=1.0,
                   want_noise=False):
  """In place on h (any shape, contiguous): h *= factor, then the dropout
  h *= (uniform < keep_prob) / keep_prob.  Returns the noise tensor when
  want_noise, else None."""
  lib = load_library()
  dt = h.dtype
  noise = torch.empty_like(h) if (want_noise and uniform is not None) else None
  with _stage("hidden_product"):
    _check(lib.mesh_moe_hidden_product(
        _dev(h, "h"),
        _dev(factor, "factor", dt, tuple(h.shape)) if factor is not None else None,
        _dev(uniform, "uniform", dt, tuple(h.shape)) if uniform is not None
        else None,
        float(keep_prob), noise.data_ptr() if noise is not None else None,
        h.numel(), dtype_code(dt), _stream()), "hidden_product")
  return noise


def expert_ffn_backward(expert_in, h, dy, wi, wo, activation="relu",
                        dh_scale=None, keep_prob=None):
  """expert_in [E,R,M], h [E,R,H], dy [E,R,N]; wi [E,M,H], wo [E,H,N] in the
  variables' own layout -> (dexpert_in [E,R,M], dwi [E,M,H], dwo [E,H,N]).
  dh_scale [E,R,H]: the hidden dropout's noise, if there was one; keep_prob:
  the keep probability it was made with (lets ReLU experts skip reading
  it)."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  e, rows, m = expert_in.shape
  hdim, n = wo.shape[1], wo.shape[2]
  dt = expert_in.dtype
  code = dtype_code(dt)
  dev = expert_in.device
  dxe = torch.empty((e, rows, m), dtype=dt, device=dev)
  dwi = torch.empty((e, m, hdim), dtype=dt, device=dev)
  dwo = torch.empty((e, hdim, n), dtype=dt, device=dev)
  ws_bytes = lib.mesh_moe_expert_ffn_backward_workspace_bytes(
      e, rows, m, hdim, n, code)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
  with _stage("expert_ffn_backward"):
    _check(lib.mesh_moe_expert_ffn_backward(
        _dev(expert_in, "expert_in"), _dev(h, "h", dt, (e, rows, hdim)),
        _dev(dy, "dy", dt, (e, rows, n)), _dev(wi, "wi", dt, (e, m, hdim)),
        _dev(wo, "wo", dt, (e, hdim, n)),
        _dev(dh_scale, "dh_scale", dt, (e, rows, hdim))
        if dh_scale is not None else None,
        float(keep_prob) if keep_prob is not None else 0.0, dxe.data_ptr(),
        dwi.data_ptr(),
        dwo.data_ptr(), e, rows, m, hdim, n, ACTIVATIONS[activation], code,
        ws.data_ptr(), ws_bytes, _stream()), "expert_ffn_backward")
  return dxe, dwi, dwo


def compact_expert_ffn_backward(expert_in, h, dy, wi, wo, r, row_offsets,
                                activation="relu", dh_scale=None,
                                keep_prob=None):
  """expert_ffn_backward with every [E, G*C, .] tensor in the compacted row
  order of compact_expert_ffn (r: the Routing, row_offsets [E, G]; dh_scale
  [E, G*C, H]: the hidden dropout's noise, if there was one)."""
  lib = load_library()
  if activation not in ("relu", "linear"):
    raise ValueError("unsupported expert activation %r" % (activation,))
  e, rows, m = expert_in.shape
  hdim, n = wo.shape[1], wo.shape[2]
  g, c = row_offsets.shape[1], r.capacity
  dt = expert_in.dtype
  dev = expert_in.device
  if rows != g * c or e != r.num_experts:
    raise MoeHipError("compact_expert_ffn_backward: expert_in is [%d, %d, .], "
                      "the routing has E=%d, G*C=%d"
                      % (e, rows, r.num_experts, g * c))
  dxe = torch.empty((e, rows, m), dtype=dt, device=dev)
  dwi = torch.empty((e, m, hdim), dtype=dt, device=dev)
  dwo = torch.empty((e, hdim, n), dtype=dt, device=dev)
  ws_bytes = lib.mesh_moe_compact_expert_ffn_backward_workspace_bytes(
      g, e, c, m, hdim, n)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("expert_ffn_backward"):
    _check(lib.mesh_moe_compact_expert_ffn_backward(
        _dev(expert_in, "expert_in"), _dev(h, "h", dt, (e, rows, hdim)),
        _dev(dy, "dy", dt, (e, rows, n)), _dev(wi, "wi", dt, (e, m, hdim)),
        _dev(wo, "wo", dt, (e, hdim, n)),
        _dev(dh_scale, "dh_scale", dt, (e, rows, hdim))
        if dh_scale is not None else None,
        float(keep_prob) if keep_prob is not None else 0.0,
        _dev(r.fill, "fill", torch.int32, (g, e)),
        _dev(row_offsets, "row_offsets", torch.int32, (e, g)), dxe.data_ptr(),
        dwi.data_ptr(), dwo.data_ptr(), g, e, c, m, hdim, n,
        ACTIVATIONS[activation], dtype_code(dt), ws.data_ptr(), ws_bytes,
        _stream()), "compact_expert_ffn_backward")
  return dxe, dwi, dwo


def expert_linear_backward(a, dy, w, want_da=True, da_relu_mask=None):
  """Backward of y = a . w per expert: a [E,R,K], dy [E,R,N], w [E,K,N] in the
  variable's own layout -> (da [E,R,K] or None, dw [E,K,N]).  da_relu_mask
  [E,R,K]: da comes out zero where the mask is not positive (the backward of
  the ReLU that made `a`, done with the product)."""
  lib = load_library()
  e, rows, k = a.shape
  n = w.shape[2]
  dt = a.dtype
  code = dtype_code(dt)
  da = torch.empty((e, rows, k), dtype=dt, device=a.device) if want_da else None
  dw = torch.empty((e, k, n), dtype=dt, device=a.device)
  ws_bytes = lib.mesh_moe_expert_linear_backward_workspace_bytes(
      e, rows, k, n, code)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=a.device)
  with _stage("expert_linear_backward"):
    _check(lib.mesh_moe_expert_linear_backward(
        _dev(a, "a"), _dev(dy, "dy", dt, (e, rows, n)),
        _dev(w, "w", dt, (e, k, n)), da.data_ptr() if want_da else None,
        dw.data_ptr(),
        None if da_relu_mask is None or not want_da else _dev(
            da_relu_mask, "da_relu_mask", dt, (e, rows, k)),
        e, rows, k, n, code, ws.data_ptr(), ws_bytes,
        _stream()), "expert_linear_backward")
  return da, dw


def activation(pre, activation):
  """act(pre), a new tensor."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  out = torch.empty_like(pre)
  with _stage("activation"):
    _check(lib.mesh_moe_activation(
        _dev(pre, "pre"), out.data_ptr(), pre.numel(), ACTIVATIONS[activation],
        dtype_code(pre.dtype), _stream()), "activation")
  return out


def activation_backward(dh, pre, activation, factor=None):
  """dh * factor * act'(pre), a new tensor of pre's shape and dtype."""
  lib = load_library()
  if activation not in ACTIVATIONS:
    raise ValueError("unsupported expert activation %r" % (activation,))
  dt = pre.dtype
  out = torch.empty_like(pre)
  with _stage("activation_backward"):
    _check(lib.mesh_moe_activation_backward(
        _dev(dh, "dh", dt, tuple(pre.shape)), _dev(pre, "pre"),
        _dev(factor, "factor", dt, tuple(pre.shape))
        if factor is not None else None,
        out.data_ptr(), pre.numel(), ACTIVATIONS[activation], dtype_code(dt),
        _stream()), "activation_backward")
  return out


def gating_backward(logits, r, dgate, d_loss, loss_scale, router="top_2",
                    importance=None, z_loss=None, num_microbatches=None,
                    importance_from_slot_gate=False, top_k=0,
                    use_second_place_loss=False, softmax_dtype=torch.float32):
  """d(logits) [G, S, E] float32.  d_loss: float32 tensor of one element on the
  device (gradient w.r.t. the layer's returned loss); loss_scale:
  moe_loss_coef.  router: "top_2", "switch" (also switch_max) or "ntlb" (then
  top_k = moe_ntlb_top_k and softmax_dtype = the forward call's)."""
  lib = load_library()
  g, s, e = logits.shape
  dev = logits.device
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  dlogits = torch.empty((g, s, e), dtype=torch.float32, device=dev)
  ws_bytes = lib.mesh_moe_gating_backward_workspace_bytes(g, e)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
  with _stage("gating_backward"):
    _check(lib.mesh_moe_gating_backward(
        _dev(logits, "logits", torch.float32), ip, icode,
        int(bool(importance_from_slot_gate)),
        _dev(r.idx, "idx", torch.int32, (g, s, 2)),
        _dev(r.kept, "kept", torch.uint8, (g, s, 2)),
        _dev(dgate, "dgate", torch.float32, (g, s, 2)),
        _dev(d_loss, "d_loss", torch.float32), float(loss_scale), g, s, e,
        {"top_2": 0, "switch": 1, "switch_max": 1, "ntlb": 2}[router],
        int(top_k), dtype_code(softmax_dtype),
        int(bool(use_second_place_loss)), int(z_loss is not None),
        float(z_loss or 0.0), int(num_microbatches or 1), dlogits.data_ptr(),
        ws.data_ptr(), ws_bytes, _stream()), "gating_backward")
  return dlogits


def router_backward_weights(x, dlogits):
  """x [T, M], dlogits [T, E] float32 -> dw_gate [M, E] of x's dtype."""
  lib = load_library()
  t, m = x.shape
  e = dlogits.shape[-1]
  out = torch.empty((m, e), dtype=x.dtype, device=x.device)
  ws_bytes = lib.mesh_moe_router_backward_weights_workspace_bytes(
      t, m, e, dtype_code(x.dtype))
  ws = torch.empty((max(ws_bytes // 4, 1),), dtype=torch.float32,
                   device=x.device)
  with _stage("router_backward_weights"):
    _check(lib.mesh_moe_router_backward_weights(
        _dev(x, "x"), _dev(dlogits, "dlogits", torch.float32, (t, e)),
        out.data_ptr(), ws.data_ptr(), t, m, e, dtype_code(x.dtype),
        _stream()), "router_backward_weights")
  return out


def dispatch_backward(dexpert_in, r, group_size, dlogits=None,
                      w_gate_packed=None, row_offsets=None, w_gate=None):
  """dexpert_in [E, G, C, M] (+ dlogits [G, S, E], w_gate_packed [B, E, M] with
  one router per G / B consecutive groups) -> dx [G, S, M].  With row_offsets
  [E, G], dexpert_in holds every expert's occupied slots first.  w_gate
  [B, M, E]: the router kernels as the variables hold them, in the activation
  dtype; with them the library may take the router's share of dx on the matrix
  cores."""
  lib = load_library()
  e, g, c, m = dexpert_in.shape
  s = group_size
  dt = dexpert_in.dtype
  dx = torch.empty((g, s, m), dtype=dt, device=dexpert_in.device)
  ip, pp, gp, kp = _routing_ptrs(r, g, s)
  dlp = wgp = wgv = None
  gpr = g
  if dlogits is not None:
    dlp = _dev(dlogits, "dlogits", torch.float32, (g, s, e))
    if w_gate_packed.dim() == 2:
      w_gate_packed = w_gate_packed.reshape(1, e, m)
    routers = w_gate_packed.shape[0]
    if g % routers:
      raise MoeHipError("dispatch_backward: %d groups, %d routers" % (g, routers))
    gpr = g // routers
    wgp = _dev(w_gate_packed, "w_gate_packed", dt, (routers, e, m))
    if w_gate is not None:
      if w_gate.dim() == 2:
        w_gate = w_gate.reshape(1, m, e)
      wgv = _dev(w_gate, "w_gate", dt, (routers, m, e))
  with _stage("dispatch_backward"):
    if row_offsets is not None:
      _check(lib.mesh_moe_dispatch_backward_compact(
          _dev(dexpert_in, "dexpert_in"), ip, pp, gp, kp,
          _dev(row_offsets, "row_offsets", torch.int32, (e, g)), dlp, wgp, wgv,
          gpr, dx.data_ptr(), g, s, e, c, m, dtype_code(dt), _stream()),
          "dispatch_backward_compact")
    else:
      _check(lib.mesh_moe_dispatch_backward(
          _dev(dexpert_in, "dexpert_in"), ip, pp, gp, kp, dlp, wgp, wgv, gpr,
          dx.data_ptr(), g, s, e, c, m, dtype_code(dt), _stream()),
          "dispatch_backward")
  return dx


# ----------------------------------------------------------------------------
# expert-selection ("expert choice") gating
# ----------------------------------------------------------------------------
class SlotRouting(object):
  """Per-slot routing record written by expert_choice_gating."""

  def __init__(self, slot_token, slot_weight, tok_slot, loss, capacity,
               num_experts):
    self.slot_token, self.slot_weight = slot_token, slot_weight
    self.tok_slot, self.loss = tok_slot, loss
    self.capacity, self.num_experts = capacity, num_experts


def expert_choice_gating(logits, capacity, importance=None, normalize=True,
                         num_microbatches=None):
  """logits float32 [G, S, E] -> SlotRouting."""
  lib = load_library()
  g, s, e = logits.shape
  c = int(capacity)
  dev = logits.device
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  slot_token = torch.empty((g, e, c), dtype=torch.int32, device=dev)
  slot_weight = torch.empty((g, e, c), dtype=torch.float32, device=dev)
  tok_slot = torch.empty((g, s, e), dtype=torch.int16, device=dev)
  loss = torch.empty((1,), dtype=torch.float32, device=dev)
  ws_bytes = lib.mesh_moe_expert_choice_workspace_bytes(g, s, e, c)
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
  with _stage("expert_choice_gating"):
    _check(lib.mesh_moe_expert_choice_gating(
        _dev(logits, "logits", torch.float32), ip, icode, g, s, e, c,
        int(bool(normalize)), int(num_microbatches or 1),
        slot_token.data_ptr(), slot_weight.data_ptr(), tok_slot.data_ptr(),
        loss.data_ptr(), ws.data_ptr(), ws_bytes, _stream()),
        "expert_choice_gating")
  r = SlotRouting(slot_token, slot_weight, tok_slot, loss, c, e)
  if _timer is not None:
    _timer.routing.append(r)
  return r


def slot_dispatch(x, r):
  """x [G, S, M] -> expert_in [E, G, C, M], one token row per slot."""
  lib = load_library()
  g, s, m = x.shape
  e, c = r.num_experts, r.capacity
  out = torch.empty((e, g, c, m), dtype=x.dtype, device=x.device)
  with _stage("slot_dispatch"):
    _check(lib.mesh_moe_slot_dispatch(
        _dev(x, "x"), _dev(r.slot_token, "slot_token", torch.int32, (g, e, c)),
        out.data_ptr(), g, s, e, c, m, dtype_code(x.dtype), _stream()),
        "slot_dispatch")
  return out


def slot_combine(y, r, group_size):
  """y [E, G, C, N] -> out [G, S, N]."""
  lib = load_library()
  e, g, c, n = y.shape
  s = group_size
  out = torch.empty((g, s, n), dtype=y.dtype, device=y.device)
  with _stage("slot_combine"):
    _check(lib.mesh_moe_slot_combine(
        _dev(y, "y"), _dev(r.tok_slot, "tok_slot", torch.int16, (g, s, e)),
        _dev(r.slot_weight, "slot_weight", torch.float32, (g, e, c)),
        out.data_ptr(), g, s, e, c, n, dtype_code(y.dtype), _stream()),
        "slot_combine")
  return out


# ---- the rest of a transformer block ----------------------------------------
def broadcast_dropout(x, sizes, uniform=None, noise=None, keep_prob=1.0,
                      want_noise=False):
  """mtf.dropout with a noise_shape (ops.py:5832-5872).  x is contiguous and
  is read as [outer, mid, inner] = sizes; uniform or noise has outer * inner
  elements and is broadcast over mid.  Returns (out, noise or None)."""
  lib = load_library()
  outer, mid, inner = (int(v) for v in sizes)
  if outer * mid * inner != x.numel():
    raise MoeHipError("sizes %s do not cover %d elements"
                      % ((outer, mid, inner), x.numel()))
  if (uniform is None) == (noise is None):
    raise MoeHipError("exactly one of uniform and noise")
  dt = x.dtype
  given = uniform if uniform is not None else noise
  if given.numel() != outer * inner:
    raise MoeHipError("noise has %d elements, expected %d"
                      % (given.numel(), outer * inner))
  out = torch.empty_like(x)
  noise_out = (torch.empty_like(uniform)
               if (want_noise and uniform is not None) else None)
  with _stage("broadcast_dropout"):
    _check(lib.mesh_moe_broadcast_dropout(
        _dev(x, "x"),
        _dev(uniform, "uniform", dt) if uniform is not None else None,
        _dev(noise, "noise", dt) if noise is not None else None,
        float(keep_prob), out.data_ptr(),
        noise_out.data_ptr() if noise_out is not None else None,
        outer, mid, inner, dtype_code(dt), _stream()), "broadcast_dropout")
  return out, (noise_out if uniform is not None else noise)


def rms_norm(x, scale, epsilon=1e-6):
  """x [..., M], scale [M] of x's dtype -> x * rsqrt(mean(x^2) + eps) * scale
  (sublayer_rms_norm, transformer/transformer.py:493-516)."""
  lib = load_library()
  m = x.shape[-1]
  rows = x.numel() // m
  out = torch.empty_like(x)
  with _stage("rms_norm"):
    _check(lib.mesh_moe_rms_norm(
        _dev(x, "x"), _dev(scale, "scale", x.dtype, (m,)), out.data_ptr(),
        rows, m, float(epsilon), dtype_code(x.dtype), _stream()), "rms_norm")
  return out


def dense(x, w_packed, activation=None):
  """x [..., K] times a packed kernel [1, N, K] -> [..., N]
  (mtf.layers.dense without bias: one einsum, ops.py / layers.py:112-160)."""
  k = x.shape[-1]
  n = w_packed.shape[1]
  y = expert_linear(x.reshape(1, -1, k), w_packed, activation)
  return y.reshape(tuple(x.shape[:-1]) + (n,))


def fused_attention_applies(q, num_heads):
  """Whether the fused attention kernels take q's shape and dtype."""
  b, l, hd = q.shape
  return hd % num_heads == 0 and load_library(
      ).mesh_moe_self_attention_backward_workspace_bytes(
          b, l, num_heads, hd // num_heads, dtype_code(q.dtype), 0) > 0


def self_attention(q, k, v, num_heads, causal, sequence_id=None,
                   relative_bias=None, return_lse=False):
  """q, k, v [B, L, H*D] -> [B, L, H*D] (attention.attention with float32
  logits, transformer/attention.py:27-88); sequence_id [B, L] int32 or None:
  a query sees only keys of its own sequence
  (transformer/transformer_layers.py:303-316).  return_lse: also the
  logarithm of the softmax denominators [B*H, L] float32 for
  self_attention_backward (fused kernels only, see fused_attention_applies)."""
  lib = load_library()
  b, l, hd = q.shape
  if hd % num_heads:
    raise MoeHipError("q channels %d not divisible by %d heads"
                      % (hd, num_heads))
  d = hd // num_heads
  code = dtype_code(q.dtype)
  out = torch.empty_like(q)
  lse = None
  if return_lse:
    lse = torch.empty((b * num_heads, l), dtype=torch.float32, device=q.device)
  ws_bytes = lib.mesh_moe_self_attention_workspace_bytes(
      b, l, num_heads, d, code, int(relative_bias is not None))
  ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=q.device)
  with _stage("self_attention"):
    _check(lib.mesh_moe_self_attention(
        _dev(q, "q"), _dev(k, "k", q.dtype, (b, l, hd)),
        _dev(v, "v", q.dtype, (b, l, hd)), out.data_ptr(), b, l, num_heads, d,
        int(bool(causal)), _sequence_id_ptr(sequence_id, b, l),
        *_relative_bias_ptrs(relative_bias, q.dtype, num_heads, l),
        None if lse is None else lse.data_ptr(), code,
        ws.data_ptr(), ws_bytes, _stream()), "self_attention")
  return (out, lse) if return_lse else out


def attention_decode(q, k_new, v_new, k_cache, v_cache, position, num_heads,
                     relative_bias=None):
  """One decoding step: q, k_new, v_new [B, H*D], the caches [B, Lm, H*D]
  (UPDATED IN PLACE at row position[b]), position [B] int32 -> out [B, H*D];
  relative_bias = (values [H, NB], bucket [2 Lm - 1] int32) or None."""
  lib = load_library()
  b, hd = q.shape
  lm = k_cache.shape[1]
  if hd % num_heads:
    raise MoeHipError("q channels %d not divisible by %d heads"
                      % (hd, num_heads))
  out = torch.empty_like(q)
  with _stage("attention_decode"):
    _check(lib.mesh_moe_attention_decode(
        _dev(q, "q"), _dev(k_new, "k_new", q.dtype, (b, hd)),
        _dev(v_new, "v_new", q.dtype, (b, hd)),
        _dev(k_cache, "k_cache", q.dtype, (b, lm, hd)),
        _dev(v_cache, "v_cache", q.dtype, (b, lm, hd)),
        _dev(position, "position", torch.int32, (b,)), out.data_ptr(), b, lm,
        num_heads, hd // num_heads,
        *_relative_bias_ptrs(relative_bias, q.dtype, num_heads, lm),
        dtype_code(q.dtype), _stream()), "attention_decode")
  return out


def slot_combine_backward(dout, y, r):
  """dout [G,S,N], y [E,G,C,N], r a SlotRouting -> (dy [E,G,C,N],
  dweight [G,E,C] float32)."""
  lib = load_library()
  e, g, c, n = y.shape
  s = dout.shape[1]
  dt = y.dtype
  dy = torch.empty_like(y)
  dweight = torch.empty((g, e, c), dtype=torch.float32, device=y.device)
  with _stage("slot_combine_backward"):
    _check(lib.mesh_moe_slot_combine_backward(
        _dev(dout, "dout", dt, (g, s, n)), _dev(y, "y"),
        _dev(r.slot_token, "slot_token", torch.int32, (g, e, c)),
        _dev(r.slot_weight, "slot_weight", torch.float32, (g, e, c)),
        dy.data_ptr(), dweight.data_ptr(), g, s, e, c, n, dtype_code(dt),
        _stream()), "slot_combine_backward")
  return dy, dweight


def slot_dispatch_backward(dxe, r, group_size, dlogits=None,
                           w_gate_packed=None, w_gate=None):
  """dxe [E,G,C,M] -> dx [G,S,M]; with dlogits [G,S,E] float32 and the packed
  router kernel [E,M] the router's share is added.  w_gate [M,E]: the kernel
  as the variable holds it (activation dtype), for the matrix-core kernel."""
  lib = load_library()
  e, g, c, m = dxe.shape
  s = group_size
  dt = dxe.dtype
  dx = torch.empty((g, s, m), dtype=dt, device=dxe.device)
  with _stage("slot_dispatch_backward"):
    _check(lib.mesh_moe_slot_dispatch_backward(
        _dev(dxe, "dxe"),
        _dev(r.tok_slot, "tok_slot", torch.int16, (g, s, e)),
        _dev(dlogits, "dlogits", torch.float32, (g, s, e))
        if dlogits is not None else None,
        _dev(w_gate_packed, "w_gate_packed", dt, (e, m))
        if w_gate_packed is not None else None,
        _dev(w_gate, "w_gate", dt, (m, e))
        if (w_gate is not None and dlogits is not None) else None,
        dx.data_ptr(), g, s, e, c, m, dtype_code(dt), _stream()),
        "slot_dispatch_backward")
  return dx


def expert_choice_backward(logits, r, dweight, d_loss, loss_scale,
                           importance=None, normalize=True,
                           num_microbatches=None):
  """d(logits) [G,S,E] float32 of expert_choice_gating."""
  lib = load_library()
  g, s, e = logits.shape
  c = r.capacity
  ip, icode = None, F32
  if importance is not None:
    icode = dtype_code(importance.dtype)
    ip = _dev(importance, "importance", None, (g, s))
  dlogits = torch.empty((g, s, e), dtype=torch.float32, device=logits.device)
  ws_bytes = lib.mesh_moe_expert_choice_backward_workspace_bytes(g, s, e)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=logits.device)
  with _stage("expert_choice_backward"):
    _check(lib.mesh_moe_expert_choice_backward(
        _dev(logits, "logits", torch.float32), ip, icode,
        _dev(r.tok_slot, "tok_slot", torch.int16, (g, s, e)),
        _dev(dweight, "dweight", torch.float32, (g, e, c)),
        _dev(d_loss, "d_loss", torch.float32, (1,)), float(loss_scale), g, s, e,
        c, int(bool(normalize)), int(num_microbatches or 1),
        dlogits.data_ptr(), ws.data_ptr(), ws_bytes, _stream()),
        "expert_choice_backward")
  return dlogits


# ---- backward of the block's operations ----------------------------------------
def rms_norm_backward(x, scale, dy, epsilon=1e-6):
  """Backward of rms_norm: x, dy [..., M], scale [M] -> (dx, dscale)."""
  lib = load_library()
  m = x.shape[-1]
  rows = x.numel() // m
  dt = x.dtype
  dx = torch.empty_like(x)
  dscale = torch.empty_like(scale)
  ws_bytes = lib.mesh_moe_rms_norm_backward_workspace_bytes(rows, m)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=x.device)
  with _stage("rms_norm_backward"):
    _check(lib.mesh_moe_rms_norm_backward(
        _dev(x, "x"), _dev(scale, "scale", dt, (m,)),
        _dev(dy, "dy", dt, tuple(x.shape)), dx.data_ptr(), dscale.data_ptr(),
        rows, m, float(epsilon), dtype_code(dt), ws.data_ptr(), ws_bytes,
        _stream()), "rms_norm_backward")
  return dx, dscale


def dense_backward(x, w, dy, y=None, want_dx=True, dx_relu_mask=False):
  """Backward of y = act(x . w): x [..., K], w [K, N] in the variable's own
  layout, dy [..., N]; with `y` (the forward output) the activation was relu.
  dx_relu_mask: x is itself the output of a ReLU whose backward is wanted on
  dx (zero where x is not positive).  Returns (dx or None, dw [K, N])."""
  k = x.shape[-1]
  n = w.shape[-1]
  x3 = x.reshape(1, -1, k)
  dy3 = dy.reshape(1, -1, n)
  if y is not None:     # relu: y > 0 exactly where the pre-activation is
    dy3 = activation_backward(dy3.contiguous(), y.reshape(1, -1, n), "relu")
  x3 = x3.contiguous()
  dx, dw = expert_linear_backward(x3, dy3.contiguous(),
                                  w.reshape(1, k, n).contiguous(),
                                  want_da=want_dx,
                                  da_relu_mask=x3 if dx_relu_mask else None)
  return (dx.reshape(x.shape) if want_dx else None), dw.reshape(k, n)


def _sequence_id_ptr(sequence_id, b, l):
  """Device pointer of sequence ids [B, L] int32, or None."""
  if sequence_id is None:
    return None
  return _dev(sequence_id, "sequence_id", torch.int32, (b, l))


def _relative_bias_ptrs(relative_bias, dtype, num_heads, l):
  """relative_bias = (values [H, NB] of the activation dtype, bucket [2L-1]
  int32) or None -> (values pointer, bucket pointer, NB)."""
  if relative_bias is None:
    return None, None, 0
  values, bucket = relative_bias
  nb = values.shape[-1]
  return (_dev(values, "relative bias values", dtype, (num_heads, nb)),
          _dev(bucket, "relative bias buckets", torch.int32, (2 * l - 1,)), nb)


def attention_weights(q, k, num_heads, causal, sequence_id=None,
                      relative_bias=None):
  """q, k [B, L, H*D] -> softmax(q . k + visibility) [B*H, L, L] in q's dtype;
  sequence_id [B, L] int32: keys of other sequences are not visible;
  relative_bias = (values [H, NB], bucket [2L-1] int32): the relative attention
  bias values[h][bucket[j - i + L - 1]] is added to logit (i, j)."""
  lib = load_library()
  b, l, hd = q.shape
  d = hd // num_heads
  code = dtype_code(q.dtype)
  weights = torch.empty((b * num_heads, l, l), dtype=q.dtype, device=q.device)
  ws_bytes = lib.mesh_moe_attention_weights_workspace_bytes(b, l, num_heads, d,
                                                            code)
  ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q.device)
  with _stage("attention_weights"):
    _check(lib.mesh_moe_attention_weights(
        _dev(q, "q"), _dev(k, "k", q.dtype, (b, l, hd)), weights.data_ptr(), b,
        l, num_heads, d, 1 if causal else 0, _sequence_id_ptr(sequence_id, b, l),
        *_relative_bias_ptrs(relative_bias, q.dtype, num_heads, l),
        code, ws.data_ptr(), ws_bytes, _stream()), "attention_weights")
  return weights


def softmax_backward(weights, dweights):
  """dlogits = w * (dw - sum_k dw * w) over the last dim."""
  lib = load_library()
  l = weights.shape[-1]
  out = torch.empty_like(weights)
  with _stage("softmax_backward"):
    _check(lib.mesh_moe_softmax_backward(
        _dev(weights, "weights"),
        _dev(dweights, "dweights", weights.dtype, tuple(weights.shape)),
        out.data_ptr(), weights.numel() // l, l, dtype_code(weights.dtype),
        _stream()), "softmax_backward")
  return out


def relative_bias_backward(dlogits, bucket, num_heads, num_buckets):
  """dlogits [B*H, L, L], bucket [2L-1] int32 -> dvalues [H, NB] (dlogits'
  dtype): the sum of dlogits over the batch and every bucket's pairs."""
  lib = load_library()
  bh, l, _ = dlogits.shape
  out = torch.empty((num_heads, num_buckets), dtype=dlogits.dtype,
                    device=dlogits.device)
  ws = torch.empty((num_heads * num_buckets,), dtype=torch.float32,
                   device=dlogits.device)
  with _stage("relative_bias_backward"):
    _check(lib.mesh_moe_relative_bias_backward(
        _dev(dlogits, "dlogits"), _dev(bucket, "bucket", torch.int32, (2 * l - 1,)),
        out.data_ptr(), ws.data_ptr(), bh // num_heads, l, num_heads,
        num_buckets, dtype_code(dlogits.dtype), _stream()),
        "relative_bias_backward")
  return out


def self_attention_backward(q, k, v, dout, num_heads, causal, fused=None,
                            sequence_id=None, relative_bias=None, out=None,
                            lse=None):
  """Backward of self_attention: q, k, v, dout [B, L, H*D] -> (dq, dk, dv).
  Shapes the fused kernels take (bf16, d_kv 64 or 128, L a multiple of 8) run
  mesh_moe_self_attention_backward: nothing [L, L] reaches memory.  Otherwise
  (or with fused=False) the weights are recomputed ([B*H, L, L]) and every
  product runs on the grouped GEMM with one (batch, head) pair per group:
    dweights = dout . v^T,  dv = weights^T . dout    (one linear backward)
    dlogits  = softmax backward
    dq = dlogits . k,       dk = dlogits^T . q
  with heads moved to the front and back by torch permutes.  fused=True raises
  for shapes the fused kernels do not take.  With relative_bias = (values
  [H, NB], bucket [2L-1]) the gradient of the values is the fourth result.
  out, lse: what self_attention(..., return_lse=True) returned for the same
  arguments; the fused kernels then skip the pass that recomputes them."""
  b, l, hd = q.shape
  h = num_heads
  if hd % h:
    raise MoeHipError("q channels %d not divisible by %d heads" % (hd, h))
  d = hd // h
  if fused is None or fused:
    lib = load_library()
    code = dtype_code(q.dtype)
    ws_bytes = lib.mesh_moe_self_attention_backward_workspace_bytes(
        b, l, h, d, code, int(relative_bias is not None))
    if ws_bytes:
      ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q.device)
      dq, dk, dv = (torch.empty_like(q) for _ in range(3))
      dvalues = None
      if relative_bias is not None:
        dvalues = torch.empty_like(relative_bias[0])
      with _stage("self_attention_backward"):
        _check(lib.mesh_moe_self_attention_backward(
            _dev(q, "q"), _dev(k, "k", q.dtype, (b, l, hd)),
            _dev(v, "v", q.dtype, (b, l, hd)),
            _dev(dout, "dout", q.dtype, (b, l, hd)), dq.data_ptr(),
            dk.data_ptr(), dv.data_ptr(), b, l, h, d, int(bool(causal)),
            _sequence_id_ptr(sequence_id, b, l),
            *_relative_bias_ptrs(relative_bias, q.dtype, h, l),
            None if dvalues is None else dvalues.data_ptr(),
            None if lse is None else _dev(out, "out", q.dtype, (b, l, hd)),
            None if lse is None else _dev(lse, "lse", torch.float32, (b * h, l)),
            code, ws.data_ptr(), ws_bytes, _stream()), "self_attention_backward")
      return (dq, dk, dv) if dvalues is None else (dq, dk, dv, dvalues)
    if fused:
      raise MoeHipError("self_attention_backward: the fused kernels do not take "
                        "dtype %s, L=%d, d_kv=%d" % (q.dtype, l, d))
  def heads_first(t):
    return t.reshape(b, l, h, d).permute(0, 2, 1, 3).reshape(b * h, l, d) \
        .contiguous()
  def heads_last(t):
    return t.reshape(b, h, l, d).permute(0, 2, 1, 3).reshape(b, l, hd) \
        .contiguous()
  qh, kh, vh, doh = (heads_first(t) for t in (q, k, v, dout))
  weights = attention_weights(q, k, h, causal, sequence_id, relative_bias)
  dweights, dvh = expert_linear_backward(weights, doh, vh)
  dlogits = softmax_backward(weights, dweights)
  del weights, dweights
  dqh = expert_linear(dlogits, pack_weights(kh, q.dtype))
  _, dkh = expert_linear_backward(dlogits, qh, vh, want_da=False)
  grads = (heads_last(dqh), heads_last(dkh), heads_last(dvh))
  if relative_bias is None:
    return grads
  values, bucket = relative_bias
  return grads + (relative_bias_backward(dlogits, bucket, h, values.shape[-1]),)
