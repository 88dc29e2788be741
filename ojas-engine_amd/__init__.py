"""MI355X (gfx950) backend for Ojas Engine's quantized-matmul path.

The directory name carries a hyphen, so import it through `__graft_entry__.load_package()`,
which registers it as the module `ojas_engine_amd`.

  runtime  — ctypes binding of libojas_hip.so shaped like the reference's Device/KernelRuntime
             and Lin/mm interfaces
  synth    — seeded synthetic tensors (benchmark distributions and the reference tests' generators)
  build    — offline build of the gfx950 code objects and the shared library
"""
from . import runtime, synth  # noqa: F401
from .runtime import (ACT_AUTO, ACT_FLOAT, ACT_FLOAT_EXACT, ACT_Q8K, ACT_Q8_1, GRID_TYPES, IQ1_M, IQ1_S, IQ2_S, IQ2_XS, IQ2_XXS, IQ3_S, IQ3_XXS, IQ4_NL, IQ4_XS, MXFP4, Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, X_BF16, X_F32, ExpertCache, Gguf, HipGpu, Lin,  # noqa: F401
                      OjasHipError, load_library, manifest, row_bytes)
