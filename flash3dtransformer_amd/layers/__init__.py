from .buck_swin import BucketSwinAttentionModule
from .elem_wise import MLP
from .flash3d import Flash3D, F3DLevelSpecs
from .hourglass import PoolingWrapper, AdditiveUnpoolingWrapper, HourglassModule
from .nn_ops import LayerNorm, LayerNormMLP, Linear, refresh_weights
from .psh_ops import PSHScatterLayer, PSH3DCoordEmbedding
from .stage import XFMRSpecs, XFMR, Stage

__all__ = [
    "AdditiveUnpoolingWrapper", "BucketSwinAttentionModule", "F3DLevelSpecs", "Flash3D", "HourglassModule",
    "LayerNorm", "LayerNormMLP", "Linear", "MLP", "PoolingWrapper", "PSH3DCoordEmbedding", "PSHScatterLayer",
    "Stage", "XFMR", "XFMRSpecs", "refresh_weights",
]
