"""MI355X-native fused expert gather / scatter-with-linear (drop-in for the reference ``egs``)."""
from .torch_interface import ExpertGather, ExpertScatter

__all__ = ["ExpertGather", "ExpertScatter"]
