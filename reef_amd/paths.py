import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
BUILD_DIR = os.path.join(CSRC_DIR, "build")
LIB_PATH = os.path.join(BUILD_DIR, "libreef_amd.so")


def code_object(flavour):
    """Path of the built code object for flavour 'raw' | 'be' | 'trans'."""
    assert flavour in ("raw", "be", "trans")
    return os.path.join(BUILD_DIR, "reef_kernels.%s.co" % flavour)
