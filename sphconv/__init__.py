"""Import path of the reference: ``import sphconv``, ``from sphconv.sphconv_cuda import get_rules``,
``from sphconv.functional import ConvFunction`` ... resolve to the modules of ``sphconv_amd`` (the same
module objects, registered under the reference's names), so code written against reveriel/sphconv
(sphconv/functional.py:7-9, sphconv/conv.py:9-14, test/test_rules.py:6-9) runs with its import lines
unchanged."""
import importlib
import sys

import sphconv_amd as _impl

_SUBMODULES = ("sphconv_cuda", "functional", "conv", "modules", "tensor", "rangevoxel", "data", "datagen", "vfe",
               "utils", "rulebook", "pipeline", "voxelize", "synth")
for _name in _SUBMODULES:
    _mod = importlib.import_module("sphconv_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    globals()[_name] = _mod
# the reference keeps its voxelisers in the package sphconv.utils (utils/voxel_generator.py, utils/voxelize.py);
# here they live in one module
sys.modules[__name__ + ".utils.voxel_generator"] = voxelize    # noqa: F821
sys.modules[__name__ + ".utils.voxelize"] = voxelize           # noqa: F821
utils.voxel_generator = voxelize                               # noqa: F821
utils.voxelize = voxelize                                      # noqa: F821

for _name in _impl.__all__:
    globals()[_name] = getattr(_impl, _name)
__all__ = list(_impl.__all__)
