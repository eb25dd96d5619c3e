"""Mirror of the reference's python/pypto/experimental package, for the operators on the sparse-attention path."""
from .gather import gather_in_l1, gather_in_ub, paged_gather

__all__ = ["gather_in_l1", "gather_in_ub", "paged_gather"]
