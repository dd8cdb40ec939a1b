from .default_hooks import _allreduce_sum_fut, dummy_hook, VSWPeerState
from .iidp_allreduce import IIDPState, iidp_allreduce_hook
from .similarity_allreduce import (GradientSimilarityState, subgroup_allreduce_hook, similimarity_allreduce_hook,
                                   cosine_similarity_from_placeholder)

__all__ = ["_allreduce_sum_fut", "dummy_hook", "VSWPeerState", "IIDPState", "iidp_allreduce_hook",
           "GradientSimilarityState", "subgroup_allreduce_hook", "similimarity_allreduce_hook",
           "cosine_similarity_from_placeholder"]
