"""Model families.  ``model_class(cfg)`` maps a configuration to the class that runs it."""


def model_class(cfg):
    family = getattr(cfg, "family", "llama")
    if family == "bozevik":
        from .bozevik import BozevikLM

        return BozevikLM
    if family == "lemunex":
        from .lemunex import LemunexLM

        return LemunexLM
    if family == "komazen":
        from .komazen import KomazenLM

        return KomazenLM
    if family == "dalalix":
        from .dalalix import DalalixLM

        return DalalixLM
    if family == "llama":
        from .transformer import TransformerLM

        return TransformerLM
    raise KeyError(f"no model class for family {family!r}")
