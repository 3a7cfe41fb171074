"""sphconv for MI355X: the sparse-convolution hot path of reveriel/sphconv
(rule generation + gather-GEMM-scatter convolution) on hand-written HIP kernels
behind the reference's Python API.  ``import sphconv_amd as sphconv``."""
from .conv import Conv3d, SparseConv3d, SubMConv3d
from .data import VoxelGenerator, merge_rangevoxel_batch, xyz2RangeVoxel
from .modules import Sequential, SparseSequential, SphModule
from .pipeline import ScanPipeline
from .rangevoxel import RangeVoxel
from .rulebook import RuleBook
from .tensor import SparseConvTensor
from ._lib import SphconvError

__all__ = ["VoxelGenerator", "merge_rangevoxel_batch", "xyz2RangeVoxel", "Conv3d", "SparseConv3d", "SubMConv3d", "Sequential", "SparseSequential", "SphModule",
           "RangeVoxel", "RuleBook", "ScanPipeline", "SparseConvTensor", "SphconvError"]
