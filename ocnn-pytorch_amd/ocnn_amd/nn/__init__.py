from .octree_pad import octree_pad, octree_depad
from .octree2col import octree2col, col2octree
from .octree_conv import (OctreeConv, OctreeDeconv, OctreeConvBase, octree_conv, octree_deconv,
                          conv_gather, conv_wgrad, column_sum)
from .octree_dwconv import OctreeDWConv, octree_dwconv
from .octree_gconv import OctreeGroupConv
from .octree_conv_t import (OctreeConvTriton, OctreeConvT, octree_conv_triton,
                            convert_conv_triton, conv_fwd_implicit_gemm_splitk,
                            conv_bwd_implicit_gemm_splitk)
from .batchnorm import BatchNormRelu1d
from .octree_pool import (octree_max_pool, octree_max_unpool, OctreeMaxPool, OctreeMaxUnpool,
                          octree_avg_pool, octree_global_pool, OctreeAvgPool, OctreeGlobalPool)
from .octree_interp import (octree_nearest_pts, octree_linear_pts, OctreeInterp,
                            octree_nearest_upsample, OctreeUpsample)

__all__ = ['octree_pad', 'octree_depad', 'octree2col', 'col2octree', 'OctreeConv', 'OctreeDeconv', 'octree_conv',
           'octree_deconv', 'OctreeDWConv', 'octree_dwconv', 'OctreeConvTriton', 'OctreeConvT',
           'octree_conv_triton', 'convert_conv_triton', 'conv_fwd_implicit_gemm_splitk',
           'conv_bwd_implicit_gemm_splitk', 'octree_max_pool', 'octree_max_unpool', 'OctreeMaxPool',
           'OctreeMaxUnpool', 'octree_nearest_pts', 'octree_linear_pts', 'OctreeInterp',
           'octree_nearest_upsample', 'OctreeUpsample', 'BatchNormRelu1d', 'octree_avg_pool',
           'octree_global_pool', 'OctreeAvgPool', 'OctreeGlobalPool', 'OctreeGroupConv']
