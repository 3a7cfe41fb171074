"""Code written against the reference runs with its import lines unchanged: ``import sphconv``,
``from sphconv.sphconv_cuda import ...`` (test/test_conv.py:5-9, sphconv/functional.py:7-9, sphconv/conv.py:9-14
of reveriel/sphconv).  The call sequence below is the one the reference's own tests use (tensor from COO
indices -> get_rules[_subm] with tile [2,2] -> rule_conv on the padded rules -> dense()); the expected values
come from torch's dense conv3d in float64, since the reference's oracle (spconv) does not exist here."""
import numpy as np
import pytest
import torch

import helpers as H

# the reference's import lines, as they stand in its tests and modules
import sphconv
from sphconv.datagen import merge_batch_torch
from sphconv.sphconv_cuda import get_rules, get_rules_subm, rule_conv
from sphconv.utils import out_spatial, voxel_generator
from sphconv.functional import ConvFunction
from sphconv.sphconv_cuda import (rule_conv_backward, to_dense, to_dense_backward, init_tensor,
                                  init_tensor_backward)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_the_alias_is_the_implementation():
    import sphconv_amd
    assert sphconv.SparseConvTensor is sphconv_amd.SparseConvTensor
    assert sphconv.sphconv_cuda is sphconv_amd.sphconv_cuda and ConvFunction is sphconv_amd.functional.ConvFunction
    assert voxel_generator.VoxelGeneratorV3 is sphconv_amd.voxelize.VoxelGeneratorV3
    for fn in (rule_conv_backward, to_dense, to_dense_backward, init_tensor, init_tensor_backward, merge_batch_torch):
        assert callable(fn)


@pytest.mark.parametrize("subm", [True, False])
def test_reference_style_call_sequence(subm):
    rng = np.random.default_rng(12)
    batch_size, spatial_shape_DWH, in_channels, out_channels = 2, [9, 14, 11], 16, 32
    kernel_size, stride, padding, dilation = [3, 3, 3], ([1, 1, 1] if subm else [2, 2, 2]), [1, 1, 1], [1, 1, 1]
    idx = np.argwhere(rng.random((batch_size, *spatial_shape_DWH)) < 0.2).astype(np.int32)
    feat = rng.standard_normal((idx.shape[0], in_channels)).astype(np.float32)
    weight = (rng.standard_normal((*kernel_size, in_channels, out_channels)) * 0.1).astype(np.float32)
    indices_bzyx = torch.tensor(idx, device=DEV)
    feature = torch.tensor(feat, device=DEV)
    w = torch.tensor(weight, device=DEV)

    tensor = sphconv.SparseConvTensor(feature, spatial_shape_DWH, batch_size, indices=indices_bzyx)
    out_spatial_shape_DWH = spatial_shape_DWH if subm else out_spatial(spatial_shape_DWH, kernel_size, stride, padding,
                                                                        dilation)
    get_rule_func = get_rules_subm if subm else get_rules
    oz_idx, oz_ptr, rules, rule_size = get_rule_func(tensor.z_idx, tensor.z_ptr, batch_size, spatial_shape_DWH,
                                                     out_spatial_shape_DWH, kernel_size, stride, padding, dilation, [2, 2])
    assert rules.dim() == 4 and rules.shape[2] == 2 and tuple(rule_size.shape) == tuple(rules.shape[:2])
    out_feature = rule_conv(tensor.feature, w.reshape(-1, in_channels, out_channels), rules, rule_size, oz_idx.shape[0])
    assert out_feature.dim() == 2 and out_feature.shape[0] == oz_idx.shape[0]
    dense = sphconv.SparseConvTensor(out_feature, out_spatial_shape_DWH, batch_size, z_ptr=oz_ptr,
                                     z_idx=oz_idx).dense(tensor.device)
    # float64 dense convolution (weight permuted as the reference does for torch, test/test_grad.py:29-36)
    x = H.dense_from_rows(feat, idx, batch_size, spatial_shape_DWH)
    want = H.dense_conv(x, weight, stride, padding, out_spatial_shape_DWH)
    if subm:
        occ = torch.zeros((batch_size, 1, *spatial_shape_DWH), dtype=torch.float64)
        occ[idx[:, 0], 0, idx[:, 1], idx[:, 2], idx[:, 3]] = 1
        want = want * occ
    assert tuple(dense.shape) == tuple(want.shape)
    torch.testing.assert_close(dense.double().cpu(), want, rtol=1e-4, atol=1e-5)
