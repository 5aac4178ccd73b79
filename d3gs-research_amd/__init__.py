"""MI355X-native 3D Gaussian splatting rasterizer (forward + backward).

Python surface of the reference's rasterize operator over hand-written gfx950
HIP kernels in ``csrc/`` (C ABI in ``include/d3gs_hip.h``).
"""
from .config_def import EarlyFilterAlgo, GaussianSplatConfig, RasterizeBackwardAlgo  # noqa: F401
from .camera import BasicPinholeCamera, Pose  # noqa: F401
from .model import GaussianModelOrigin, GaussianModelOriginBase, GaussianModelOriginFused  # noqa: F401


def __getattr__(name):
    # render imports torch and loads the HIP library; keep `import package` light
    if name in ("GaussianSplatOp", "GaussianSplatOutput", "GaussianSplatOpContext", "GaussianSplatGradients",
                "RasterizeGradientOutput", "CameraBundle", "rasterize_gaussians"):
        from . import render
        return getattr(render, name)
    raise AttributeError(name)
