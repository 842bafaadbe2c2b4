"""Modifier registry, as spotlight/modifiers/__init__.py:1-44 for the generation
methods this package implements."""


def get_modifier(method: str, model_type: str = None):
    if method in ("spotlight-generation", "spotlight-generation-hip"):
        from .spotlight_generation import Spotlight
        return None, Spotlight
    if method in ("linearhashing-generation", "linearhashing-generation-hip"):
        from .linearhashing_generation import LinearHashing
        return None, LinearHashing
    raise NotImplementedError(method, model_type)
