from .gs_2d_render import GS_2D_render, GS_2D_topk_weights, GS_prepare, RasterizeBuffer, render_step  # noqa: F401
from .gs_2d_fast_render import (GS_2D_fast_render, GS_2D_fast_preprocess, GS_2D_fast_rasterize,  # noqa: F401
                                GS_2D_fast_rasterize_v2, fast_compuate_transmat, fast_render_step)
from . import gaussian_render  # noqa: F401  (3D-Gaussian path: gaussian_render.render, .preprocess, .GS_render)
