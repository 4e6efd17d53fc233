"""An LFM2 inference engine for one AMD MI355X (gfx950).

The package is assembled from independent subsystems:

  config/    typed configurations and the architecture registry
  weights/   safetensors reading/writing, by-name loading, random model folders
  parts/     mixers, feed-forwards, norms, position encodings, block arrangements
  cache/     paged key/value pools, block tables, fixed-size state slots
  engine/    the step function, the scheduler and the generation loop
  sampling/  greedy / temperature / top-k / top-p / repetition penalty
  kernels/   Python bindings of the HIP kernels under csrc/
  csrc/      hand-written HIP sources for gfx950

Importing the package touches neither the GPU nor the compiler; kernels are
compiled and loaded the first time one of them is called.
"""

__version__ = "0.1.0"

from .config import load_config, register_architecture, known_architectures  # noqa: F401


def __getattr__(name):
    # The engine classes import torch-heavy modules; load them on first use.
    if name in ("Engine", "DecoderModel", "ModelRunner", "StepEntry", "Scheduler", "Request"):
        from . import engine
        return getattr(engine, name)
    if name in ("SamplingParams",):
        from . import sampling
        return getattr(sampling, name)
    raise AttributeError(name)
