from .gs_2d_render import GS_2D_render, GS_2D_topk_weights, GS_prepare, RasterizeBuffer, render_step  # noqa: F401
