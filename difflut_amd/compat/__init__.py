"""Modules with the names and call signatures of the reference's pybind extensions
(mapping_cuda, efd_cuda, efd_fused_cuda, dwn_stable_cuda, hybrid_cuda, probabilistic_cuda,
learnable_mapping_cuda), implemented
on libdifflut_hip.so.  Put this directory on sys.path (difflut_amd.compat.install()) and the
reference's own `import efd_cuda` style imports (difflut/nodes/dwn_node.py:31-55,
difflut/layers/random_layer.py:17-31, ...) resolve to them."""
import os
import sys


def install():
    here = os.path.dirname(os.path.abspath(__file__))
    if here not in sys.path:
        sys.path.insert(0, here)
