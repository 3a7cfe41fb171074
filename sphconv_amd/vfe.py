"""Voxel feature encoders of the data path (reference: sphconv/vfe.py)."""
import torch
from torch import nn


class SimpleVoxel(nn.Module):
    """Mean of the points of a voxel (vfe.py:210-228)."""

    def __init__(self, num_input_features=4, use_norm=True, num_filters=(32, 128), with_distance=False,
                 voxel_size=(0.2, 0.2, 4), pc_range=(0, -40, -3, 70.4, 40, 1), name="VoxelFeatureExtractor"):
        super().__init__()
        self.name = name
        self.num_input_features = num_input_features

    def forward(self, features, num_voxels, coors):
        # features [voxels, max_points, >=num_input_features], unused slots are zero
        points_mean = features[:, :, :self.num_input_features].sum(dim=1, keepdim=False) \
            / num_voxels.type_as(features).view(-1, 1)
        return points_mean.contiguous()
