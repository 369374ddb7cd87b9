"""Rule filtering (reference: fms_acceleration_foak/utils.py:84-96).  The reference's FSDP helper
that all-reduces adapter gradients across ranks is a multi-GPU concern and is not part of this
single-GPU build."""
from typing import List, Set

from fms_acceleration.model_patcher import ModelPatcherRule


def filter_mp_rules(rules: List[ModelPatcherRule], filter_endswith: Set[str], drop: bool = False):
    """Keep (or, with drop=True, discard) the rules whose id ends with any of the given terms."""
    def hit(rule):
        return any(rule.rule_id.endswith(term) for term in filter_endswith)

    return [r for r in rules if hit(r) != drop]
