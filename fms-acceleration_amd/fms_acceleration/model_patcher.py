"""ModelPatcher: rules that rebind `module.forward` (or swap an imported symbol) on a loaded model.

Behavioural mirror of plugins/framework/src/fms_acceleration/model_patcher.py:
  * triggers fire on isinstance or on a callable; a callable that raises counts as "not
    triggered" (:92-110); an optional module_name narrows the trigger (:98-99)
  * a rule carries at most one of forward / forward_builder / import_and_maybe_reload, and
    import_and_maybe_reload excludes a trigger (:178-204)
  * rules are class-level (singleton) state, duplicate ids assert (:230-266)
  * per module the FIRST triggered rule wins; later simple-forward rules only warn (:269-293)
  * a forward_builder that returns a list of (trigger, forward) pairs is applied to that module's
    own sub-tree as temporary rules "<id>-1", "<id>-2", ... (:441-471)
  * history / summary of what was patched (:208-227, 500-524)
"""
from __future__ import annotations

import importlib
import importlib.util
import inspect
import warnings
from dataclasses import asdict, dataclass
from enum import Enum
from types import MethodType
from typing import Any, Callable, Dict, List, Optional, Set, Tuple, Type, Union

import torch


def patch_target_module(to_patch: str, replace_with: Any, target_module: str = None):
    """Set `pkg.mod.obj = replace_with`.  With `target_module`, reload that module while the
    replacement is in place (so its `from pkg.mod import obj` picks it up) and then restore the
    original object on the source module."""
    parts = to_patch.split(".")
    assert len(parts) > 1, "must have an object to patch"
    source = importlib.import_module(".".join(parts[:-1]))
    original = getattr(source, parts[-1])
    setattr(source, parts[-1], replace_with)
    if target_module is not None:
        importlib.reload(importlib.import_module(target_module))
        setattr(source, parts[-1], original)


class ModelPatcherTriggerType(Enum):
    module = 1
    callable = 2


@dataclass
class ModelPatcherTrigger:
    check: Union[Type[torch.nn.Module], Callable[[torch.nn.Module], bool]]
    type: ModelPatcherTriggerType = None
    module_name: str = None

    def __post_init__(self):
        if inspect.isclass(self.check) and issubclass(self.check, torch.nn.Module):
            inferred = ModelPatcherTriggerType.module
        elif callable(self.check):
            inferred = ModelPatcherTriggerType.callable
        else:
            raise TypeError("check argument needs to be torch.nn.Module or Callable")
        if self.type is None:
            self.type = inferred
        else:
            assert self.type == inferred, "type argument passed but `check` argument does not match type specified"

    def is_triggered(self, module: torch.nn.Module, module_name: str = None) -> bool:
        if self.module_name is not None and module_name != self.module_name:
            return False
        if self.type == ModelPatcherTriggerType.module:
            return isinstance(module, self.check)
        try:
            return bool(self.check(module))
        except Exception:  # pylint: disable=broad-exception-caught
            return False  # e.g. a check that reads attributes this module does not have


ModelForward = Callable


@dataclass
class ModelPatcherRule:
    rule_id: str
    trigger: ModelPatcherTrigger = None
    forward: ModelForward = None
    forward_builder: Callable[[torch.nn.Module], Union[ModelForward, List[Tuple[ModelPatcherTrigger, ModelForward]]]] = None
    forward_builder_args: List[str] = None
    import_and_maybe_reload: Tuple[str, Type, Optional[str]] = None

    def __post_init__(self):
        n_actions = sum(x is not None for x in (self.forward, self.forward_builder, self.import_and_maybe_reload))
        if n_actions > 1:
            raise ValueError(
                f"Rule '{self.rule_id}' must only have at most one of forward, "
                "forward builder, or import_and_maybe_reload, specified."
            )
        if self.import_and_maybe_reload is not None and self.trigger is not None:
            raise ValueError(f"Rule '{self.rule_id}' has import_and_maybe_reload specified, and trigger must be None.")
        if self.forward_builder_args is not None and self.forward_builder is None:
            raise ValueError(f"Rule '{self.rule_id}' has forward_builder_args but no forward_builder.")


@dataclass
class ModelPatcherHistory:
    instance: int
    cls: str
    parent_cls: str
    module_name: str
    parent_module_name: str
    rule_id: str


class ModelPatcher:
    history: List[ModelPatcherHistory] = []
    rules: Dict[str, ModelPatcherRule] = {}

    @staticmethod
    def load_patches(module_names: List[str], reload: bool = False):
        for name in module_names:
            if importlib.util.find_spec(name):
                m = importlib.import_module(name)
                if reload:
                    try:
                        importlib.reload(m)
                    except AssertionError:
                        pass  # its rules are registered already

    @staticmethod
    def register(rule: ModelPatcherRule):
        assert rule.rule_id not in ModelPatcher.rules, f"patch rule '{rule.rule_id}' already exists"
        ModelPatcher.rules[rule.rule_id] = rule

    @staticmethod
    def did_rule_trigger(module: torch.nn.Module, module_name: str):
        winner_id, winner = None, None
        for rule_id, rule in ModelPatcher.rules.items():
            if rule.trigger is None or not rule.trigger.is_triggered(module, module_name):
                continue
            if winner is None:
                winner_id, winner = rule_id, rule
            elif rule.forward is not None:
                warnings.warn(
                    f"rule {rule.rule_id} is ignored on {module_name} as an earlier rule {winner.rule_id} has been applied"
                )
        return winner_id, winner

    @staticmethod
    def _import_and_reload(model: torch.nn.Module):
        """Apply the trigger-less rules whose target (or reload path) lives under the model's own
        python module.  Reloading rules go first; two rules may not reload nested paths."""
        module_path = model.__module__
        reloading, plain = [], []
        for rule in ModelPatcher.rules.values():
            if rule.import_and_maybe_reload is None:
                continue
            target, _, reload_path = rule.import_and_maybe_reload
            if reload_path and reload_path.startswith(module_path):
                reloading.append(rule)
            elif target.startswith(module_path):
                plain.append(rule)
        reloading.sort(key=lambda r: len(r.import_and_maybe_reload[2]))
        for i, short in enumerate(reloading[:-1]):
            for long in reloading[i + 1:]:
                name_s, obj_s, path_s = short.import_and_maybe_reload
                path_l = long.import_and_maybe_reload[2]
                if path_s == path_l:
                    short.import_and_maybe_reload = (name_s, obj_s, None)  # reload that path once only
                    continue
                assert not path_l.startswith(path_s), (
                    f"Attempting to reload a subpath`{path_s}` multiple times in {short.rule_id} and {long.rule_id}"
                )
        for rule in reloading + plain:
            target, obj, reload_path = rule.import_and_maybe_reload
            patch_target_module(target, obj, reload_path)
            ModelPatcher.history.append(
                ModelPatcherHistory(id(model), model.__class__.__name__, "", "", "", rule.rule_id)
            )

    @staticmethod
    def _patch_forwards(model, patch_kwargs: Dict = None, visited: Set = None, parent_prefix: str = None,
                        parent_mcn: str = None):
        patch_kwargs = patch_kwargs or {}
        visited = set() if visited is None else visited
        for full_name, mod in model.named_modules():
            parts = full_name.split(".")
            if len(parts) > 2:
                parent_name, module_name = ".".join(parts[:-1]), parts[-1]
                parent_cls = model.get_submodule(parent_name).__class__.__name__
            else:
                # the model itself and names of depth <= 2 report their first component (:414-419)
                module_name = parts[0]
                parent_name, parent_cls = "", ""
                if parent_prefix is not None:
                    parent_name = parent_prefix + "." + parent_name
                if parent_mcn is not None:
                    parent_cls = parent_mcn

            rule_id, rule = ModelPatcher.did_rule_trigger(mod, module_name)
            if rule_id is None:
                continue
            if rule.forward is not None:
                forward = rule.forward
            elif rule.forward_builder is not None:
                extra = {}
                if rule.forward_builder_args is not None:
                    extra = {k: v for k, v in patch_kwargs.items() if k in rule.forward_builder_args}
                forward = rule.forward_builder(mod, **extra)
            else:
                forward = None  # trigger-only rule: recorded in the history, nothing rebound

            if isinstance(forward, list):
                saved = ModelPatcher.rules
                ModelPatcher.rules = {}
                try:
                    for i, (trig, fwd) in enumerate(forward):
                        ModelPatcher.register(ModelPatcherRule(rule_id=f"{rule_id}-{i + 1}", trigger=trig, forward=fwd))
                    ModelPatcher._patch_forwards(mod, patch_kwargs=patch_kwargs, visited=visited,
                                                 parent_prefix=parent_name, parent_mcn=parent_cls)
                finally:
                    ModelPatcher.rules = saved
                continue

            if forward is not None:
                mod.forward = MethodType(forward, mod)
            ModelPatcher.history.append(
                ModelPatcherHistory(id(mod), mod.__class__.__name__, parent_cls, module_name, parent_name, rule_id)
            )

    @staticmethod
    def patch(model: torch.nn.Module, **kwargs):
        try:
            ModelPatcher._import_and_reload(model.get_base_model())
        except AttributeError:
            ModelPatcher._import_and_reload(model)
        ModelPatcher._patch_forwards(model, patch_kwargs=kwargs)

    @staticmethod
    def summary(raw: bool = False):
        """raw=True: the history as a pandas DataFrame; otherwise a printable table grouped by
        (rule_id, module_name, cls) with instance counts."""
        if raw:
            import pandas as pd  # pylint: disable=import-outside-toplevel

            return pd.DataFrame([asdict(h) for h in ModelPatcher.history])
        if not ModelPatcher.history:
            return ""
        counts: Dict[Tuple[str, str, str], int] = {}
        for h in ModelPatcher.history:
            key = (h.rule_id, h.module_name, h.cls)
            counts[key] = counts.get(key, 0) + 1
        lines = ["***************** Module Forwards Patching *************"]
        for (rule_id, module_name, cls), n in sorted(counts.items()):
            lines.append("Rule: {0:15s} Module: {1:25s} Class: {2:15s} Num: {3:2d}".format(rule_id, module_name, cls, n))
        return "\n".join(lines)


def patch_model(model: torch.nn.Module, **kwargs):
    ModelPatcher.patch(model, **kwargs)
    return model


def patch_model_summary():
    return ModelPatcher.summary()


def combine_triggers(*triggers: ModelPatcherTrigger, logic: str = "OR"):
    assert logic in ["AND", "OR"], "Only `AND`, `OR` logic implemented for combining triggers"
    reduce = any if logic == "OR" else all

    def _combined(*args, **kwargs):
        return reduce(t.is_triggered(*args, **kwargs) for t in triggers)

    return ModelPatcherTrigger(check=_combined)


def combine_functions(*funcs: Callable, logic: str = "APPEND"):
    assert logic == "APPEND", "only APPEND logic implemented for combining functions"

    def _append(*args, **kwargs):
        out = []
        for f in funcs:
            out += f(*args, **kwargs)
        return out

    return _append
