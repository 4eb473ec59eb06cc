"""MI355X-native implementation of the Fast-SP-GS `fast_2d_gs/_C` hot path (2D Gaussian surfel rendering and its
companion operators), behind the reference's Python-facing operator API.

    from fast_sp_gs_amd._C import get_C_function          # name -> callable, as fast_2d_gs/_C/__init__.py
    from fast_sp_gs_amd.renderer import GS_2D_render        # autograd wrapper + epilogue, as renderer/gs_2d_render.py
"""
__version__ = "0.1.0"
