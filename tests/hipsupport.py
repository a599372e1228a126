"""GPU-side test helpers: the package's session over the C-ABI library (device buffers, uploads,
step and frame calls).  Everything here calls the product through `extern "C"` entry points only."""
import os

import vtsupport as S

ROOT = S.ROOT
PKG_DIR = S.PKG_DIR
load_package = S.load_package

load_package()
from voxtral_tts_c_amd.session import DevBuf, Hip, host_layer  # noqa: E402,F401


def gpu_present():
    return os.path.exists("/dev/kfd") and os.path.isdir("/dev/dri")
