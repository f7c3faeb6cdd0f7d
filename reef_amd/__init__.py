"""reef_amd: MI355X-native REEF hot path (executors, DKP/preemptible kernels, scheduler).

The compute lives in hand-written gfx950 code objects and a C++ host library
(``csrc/``); this package holds the ctypes binding of the flat C API
(``include/reef_c.h``) and the model-directory generator (``modelgen``).
"""
from .paths import CSRC_DIR, BUILD_DIR, LIB_PATH, code_object  # noqa: F401
