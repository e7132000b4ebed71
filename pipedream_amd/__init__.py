"""pipedream_amd -- PipeDream's per-stage training step for MI355X (gfx950).

Host-side classes keep the reference's names and call signatures
(``runtime.StageRuntime``, ``optimizer.OptimizerWithWeightStashing``,
``sgd.SGDWithWeightStashing``, ``adam.AdamWithWeightStashing``); the device work is done
by hand-written HIP kernels in ``libpipedream_amd.so`` reached through a C ABI.
"""
from . import _cabi  # noqa: F401  (fails loudly if the library has not been built)

__all__ = ["_cabi"]
