"""MI355X-native top-2 Mixture-of-Experts layers behind a Mesh-TensorFlow-shaped
API.  `import mesh_amd as mtf` gives the graph vocabulary (Dimension, Shape,
Graph, Mesh, Lowering, VariableDType, ...); `mesh_amd.transformer.moe` holds the
layers; `mesh_amd.HipMeshImpl` is the single-GPU MeshImpl that runs them on
libmesh_moe_hip.so.
"""

from mesh_amd.ops import *  # pylint: disable=wildcard-import
from mesh_amd.ops import (Dimension, Shape, LayoutRules, TensorLayout, Graph,
                          Mesh, Tensor, Operation, MeshImpl, Lowering,
                          SlicewiseOperation, ReshapeOperation,
                          ImportOperation, Constant, Variable, VariableDType,
                          convert_to_dimension, convert_to_shape,
                          convert_to_layout_rules,
                          convert_args_to_laid_out_tensors,
                          tensor_dim_to_mesh_dim_size, variable_scope,
                          float32, bfloat16, int32)
from mesh_amd import layers
from mesh_amd.hip_mesh_impl import HipMeshImpl
