from .base_model import BaseModel
from .tree import Tree

__all__ = ["BaseModel", "Tree"]
