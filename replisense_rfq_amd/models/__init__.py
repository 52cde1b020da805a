"""Model classes.  Layer-list models are chosen by their configuration's architecture."""


def layered_model_class(architecture: str):
    """Model class of a layer-list architecture (imported on demand: each brings only the
    kernels it runs)."""
    if architecture == "Livisun":
        from .livisun import LivisunLM

        return LivisunLM
    if architecture == "Numalorn":
        from .numalorn import NumalornLM

        return NumalornLM
    if architecture == "Bilolix":
        from .bilolix import BilolixLM

        return BilolixLM
    if architecture == "Nutitar":
        from .nutitar import NutitarLM

        return NutitarLM
    raise KeyError(f"no model class for architecture {architecture!r}")
