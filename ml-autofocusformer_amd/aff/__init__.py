"""The callers on either side of the CLUSTEN operators: the producer of the neighbourhood lists and the two
modules that consume the operators, assembled into an AutoFocusFormer classifier for end-to-end measurement."""
from .points import knn, space_filling_cluster  # noqa: F401
