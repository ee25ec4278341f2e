"""axon_amd: a small, whole inference engine for AMD MI355X (gfx950), one GPU.

    import axon_amd
    llm = axon_amd.load("path/to/model", dtype="bfloat16")
    out = llm.generate([[1, 2, 3]], max_new_tokens=16)
"""
__version__ = "0.1.0"


def load(*args, **kwargs):
    from .engine.llm import load as _load
    return _load(*args, **kwargs)


def __getattr__(name):
    if name in ("LLM", "SamplingParams"):
        from .engine import llm
        return getattr(llm, name)
    raise AttributeError(name)
