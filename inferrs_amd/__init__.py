"""inferrs_amd: a small, whole inference engine for one AMD MI355X, in the manner of inferrs.

    config/    typed configuration from config.json, the architecture registry, layer specs
    weights/   safetensors by tensor name, load checks, random model folders
    parts/     norm, position encoding, attention, feed-forward, block: built from specs
    cache/     pages with block tables per request, per-request state slots
    engine/    model assembly, the step function, the scheduler, generation
    sampling/  sampling parameters and the device sampler
    cli.py     `inferrs-amd run | bench`, in the reference's manner
    ops/       host checks and C calls into the HIP kernels of csrc/
"""
__version__ = "0.1.0"


def __getattr__(name):
    """`inferrs_amd.Engine`, `inferrs_amd.SamplingParams`, `inferrs_amd.generate`: the Python entry
    point, loaded on first use (importing the package alone needs no GPU)."""
    if name in ("Engine", "Entry", "GenerationLoop", "generate"):
        from . import engine
        return getattr(engine, name)
    if name == "SamplingParams":
        from .sampling import SamplingParams
        return SamplingParams
    raise AttributeError(f"module 'inferrs_amd' has no attribute {name!r}")
