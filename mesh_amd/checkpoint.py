"""Loading and saving the variables of a lowered graph by name.

The variable names and shapes of the layers in this package are the
reference's, so a Mesh-TensorFlow checkpoint maps onto them one to one.  This
module restates the selection logic of the reference's initialisation from a
checkpoint (mesh_tensorflow/transformer/utils.py:947-972: optional regular
expression filter on the checkpoint's names, a graph-name -> checkpoint-name
mapping, a should-load predicate) and the two hooks around TensorFlow's saver
(mesh_tensorflow/ops.py:5740-5779: masters are copied to slices after a
restore, slices to masters before a save).

A checkpoint is a mapping name -> array, the path of a NumPy `.npz` archive of
such a mapping, the prefix of a TensorFlow tensor bundle (`model.ckpt-1000`
beside `model.ckpt-1000.index` and `.data-*`), or a directory whose `checkpoint`
file names such a prefix (mesh_amd/tensor_bundle.py reads and writes the
bundles without TensorFlow).
"""

import collections
import os
import re

import numpy as np
import torch

from mesh_amd import tensor_bundle

RestoreReport = collections.namedtuple(
    "RestoreReport",
    ["restored", "in_checkpoint_not_in_graph", "in_graph_not_in_checkpoint"])


def plan_restore(graph_names, checkpoint_names, variable_filter=None,
                 variable_mapping=None, should_load=None):
  """Which variables to restore (utils.py:948-972).

  graph_names / checkpoint_names: iterables of names.  variable_filter: a
  regular expression the CHECKPOINT names must match (init_variable_filter);
  variable_mapping: graph name -> checkpoint name (identity by default);
  should_load: predicate on graph names (everything by default).
  Returns RestoreReport(restored = {graph name: checkpoint name}, two sorted
  lists).
  """
  mapping = variable_mapping or (lambda name: name)
  should_load = should_load or (lambda name: True)
  ckpt = set(checkpoint_names)
  if variable_filter:
    pattern = re.compile(variable_filter)
    ckpt = {v for v in ckpt if pattern.search(v)}
  graph_all = set(graph_names)
  filtered = {v for v in graph_all if should_load(v)}
  restore = {v: mapping(v) for v in filtered if mapping(v) in ckpt}
  return RestoreReport(
      restore,
      sorted(ckpt - {mapping(v) for v in filtered}),
      sorted(graph_all - set(restore)))


def _open(checkpoint):
  if not isinstance(checkpoint, str):
    return checkpoint
  if os.path.isdir(checkpoint):
    prefix = tensor_bundle.latest_checkpoint(checkpoint)
    if prefix is None:
      raise ValueError("no checkpoint state file in %s" % checkpoint)
    return tensor_bundle.BundleReader(prefix)
  if os.path.exists(checkpoint + ".index"):
    return tensor_bundle.BundleReader(checkpoint)
  return np.load(checkpoint, allow_pickle=False)


def restore_variables(lowering, checkpoint, variable_filter=None,
                      variable_mapping=None, should_load=None):
  """Sets the masters of the selected variables from `checkpoint` and copies
  masters to slices (MtfRestoreHook, ops.py:5760-5779).  A shape mismatch
  raises ValueError, as tf.train.init_from_checkpoint does."""
  arrays = _open(checkpoint)
  by_name = {v.name: (v, lv) for v, lv in lowering.variables.items()}
  names = arrays.files if hasattr(arrays, "files") else list(arrays.keys())
  report = plan_restore(by_name, names, variable_filter, variable_mapping,
                        should_load)
  for graph_name, ckpt_name in sorted(report.restored.items()):
    variable, laid_out = by_name[graph_name]
    value = np.asarray(arrays[ckpt_name])
    if list(value.shape) != variable.shape.to_integer_list:
      raise ValueError(
          "checkpoint tensor %s has shape %s, variable %s has shape %s"
          % (ckpt_name, list(value.shape), graph_name,
             variable.shape.to_integer_list))
    laid_out.assign(torch.from_numpy(np.ascontiguousarray(value)))
  lowering.copy_masters_to_slices()
  return report


def save_variables(lowering, path=None):
  """Copies slices to masters (MtfCheckpointSaverListener.before_save,
  ops.py:5740-5757) and returns {name: float32 / integer NumPy array of the
  master}.  With a `path` ending in `.npz` also writes them as a NumPy
  archive; with any other `path`, as a TensorFlow tensor bundle of that prefix,
  and points the directory's `checkpoint` file at it."""
  lowering.copy_slices_to_masters()
  out = {}
  for variable, laid_out in lowering.variables.items():
    master = laid_out.master.detach()
    if master.dtype == torch.bfloat16:
      master = master.float()
    out[variable.name] = master.cpu().numpy()
  if path is not None and path.endswith(".npz"):
    np.savez(path, **out)
  elif path is not None:
    tensor_bundle.write_bundle(path, out)
    tensor_bundle.write_checkpoint_state(path)
  return out
