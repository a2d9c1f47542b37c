from .shuffled_key import key2xyz, xyz2key
from .points import Points, merge_points
from .octree import Octree, init_octree, merge_octrees
from .contract import ContractOctree, tables_of

__all__ = ['xyz2key', 'key2xyz', 'Points', 'Octree', 'merge_points', 'merge_octrees',
           'init_octree', 'ContractOctree', 'tables_of']
