"""CPU oracle for the Cosmos 3 Generator-mode DM block forward.

TEST INFRASTRUCTURE ONLY.  Nothing under ``cosmos_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may, and only as the checker.

The reference repository (NVIDIA/cosmos) holds no implementation of the block:
it names the architecture (README.md:74 and
cookbooks/cosmos3/cosmos3-model-architecture.png) and calls it through the
diffusers pipeline (README.md:238-263,
cookbooks/cosmos3/generator/audiovisual/run_with_diffusers.ipynb:523-612).
The arithmetic lives in ``diffusers`` git main (unpinned, README.md:219-229),
which is not installed here, so this oracle restates the published algorithm
from the reference's architecture text plus the operator definitions that the
installed ``transformers 5.15.0`` carries for the Cosmos 3 AR tower.

Pinning status of each oracle function
--------------------------------------
pinned by library golden vectors (tests/golden/tf_fixtures.npz) and by
closed forms / float64 brute force (tests/test_oracle_*.py):
    rms_norm, rotate-half mRoPE (chunked and interleaved tables, apply),
    vision / text position ids, attention (multi-head and grouped-query),
    swiglu, pre-norm residual wiring (also with grouped K/V heads).
pinned by closed forms and float64 brute force only (no library routine
exists for them):
    adaln_rms_norm modulation, gated residual, MoT segment routing,
    e4m3 quantisation (against torch.float8_e4m3fn casts), cfg_step (guidance
    combine + linear scheduler update); oracle/unipc.py (UniPC predictor /
    corrector updates: Euler closed form, exactness on polynomial data
    predictions against quadrature of the exact solution, convergence orders).
parity unpinned against the real Cosmos 3 generator (only an import of the
absent diffusers implementation could pin them; the benchmark configuration
text governs instead):
    timestep_embedding / time_mlp conventions, adaLN chunk order and the
    (1 + scale) convention, mRoPE channel layout choice (chunked is the
    default), modality position offsets in generator mode, the fp8 recipe,
    the scheduler as diffusers configures it (oracle/unipc.py restates the
    published UniPC algorithm; diffusers' noise-level grid, default order and
    final-step handling are restated from its documentation, not executed).
"""
from .dm_oracle import *  # noqa: F401,F403
