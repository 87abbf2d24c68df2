from .entry import IndexEntry
from .staged import IndexStaged, GraphModule

__all__ = ['IndexEntry', 'IndexStaged', 'GraphModule']
