"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol include/fsgs.h and include/fsgs_debug.h declare,
the operator namespace mirrors the reference's `fast_2d_gs/_C/__init__.py` helpers, and argument errors surface as
RuntimeError before any kernel is launched. No compute call is made here (no GPU)."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]

REFERENCE_NAMES = [  # the pybind m.def names on the hot path
    'gs_2d_preprocess_forward', 'gs_2d_preprocess_backward', 'gs_2d_compute_transmat_forward',
    'gs_2d_compute_trans_mat_backward', 'GS_prepare', 'GS_2D_render_forward', 'GS_2D_render_backward',
    'sh_encode_forward', 'sh_encode_backward', 'SH_to_RGB_forward', 'SH_to_RGB_backward', 'freq_encode_forward',
    'freq_encode_backward', 'cdist_top', 'cdist_top_backward', 'AdamMasksedUpdated',
]


def test_library_exports_every_declared_symbol():
    from fast_sp_gs_amd import lib
    text = (ROOT / "include" / "fsgs.h").read_text() + (ROOT / "include" / "fsgs_debug.h").read_text()
    declared = set(re.findall(r"\b(fsgs_\w+)\s*\(", re.sub(r"/\*.*?\*/", " ", text, flags=re.S)))
    assert len(declared) >= 26
    L = lib.load()
    for name in declared:
        assert hasattr(L, name), name
    assert set(lib.prototypes()) == declared
    assert L.fsgs_version() >= 100
    assert isinstance(L.fsgs_last_error(), bytes)


def test_workspace_queries_are_host_only():
    from fast_sp_gs_amd import lib
    L = lib.load()
    assert L.fsgs_gs_prepare_scan_workspace_bytes(300_000) >= (300_000 // 2048 + 1) * 8
    assert L.fsgs_gs_prepare_fill_workspace_bytes(1_000_000) >= 1_000_000 * 20
    assert L.fsgs_gs_prepare_sort_bits(800, 800) == 44 and L.fsgs_gs_prepare_sort_bits(256, 256) == 41
    assert L.fsgs_lbs_blend_workspace_bytes(512) >= 512 * 48


def test_operator_namespace_semantics():
    from fast_sp_gs_amd import _C
    for name in REFERENCE_NAMES:
        assert callable(_C.get_C_function(name)), name
        assert _C.have_C_functions(name)
    assert _C.get_C_function('no_such_op') is None
    assert not _C.have_C_functions('GS_prepare', 'no_such_op')
    f = lambda: None
    assert _C.get_C_function(f) is f

    # bare use: registers the python function and hands back the native one of the same name
    def GS_prepare(*a):
        return 'python'

    native = _C.try_use_C_extension(GS_prepare)
    assert native is _C.get_C_function('GS_prepare') and _C.get_python_function('GS_prepare') is GS_prepare

    # with dependencies: decorator returning the native-backed callable iff all dependencies exist
    sentinel = object()

    @_C.try_use_C_extension(sentinel, 'sh_encode_forward', 'sh_encode_backward')
    def sh_encode(*a):
        return 'python'

    assert sh_encode is sentinel
    with pytest.warns(UserWarning):
        @_C.try_use_C_extension(sentinel, 'sh_encode_forward', 'missing_dependency')
        def other(*a):
            return 'python'
    assert other() == 'python'
    with pytest.raises(AttributeError):
        _C.no_such_op


def test_argument_errors_raise_before_launch():
    from fast_sp_gs_amd._C import get_C_function
    P = 4
    cpu = lambda *s: torch.zeros(*s)
    with pytest.raises(RuntimeError, match="CUDA"):
        get_C_function('gs_2d_preprocess_forward')(64, 64, 3, False, cpu(P, 3), cpu(P, 2), cpu(P, 4), cpu(P, 1),
                                                   cpu(P, 16, 3), None, cpu(4, 4), cpu(4, 4), cpu(3), None, None, None)
    with pytest.raises(RuntimeError, match="CUDA"):
        get_C_function('GS_prepare')(64, 64, cpu(P, 2), cpu(P), torch.zeros(P, dtype=torch.int32),
                                     torch.zeros(P, dtype=torch.int32), False)
    with pytest.raises(RuntimeError):
        get_C_function('cdist_top')(cpu(5, 3), cpu(7, 3))


def test_c_abi_rejects_bad_sizes_without_touching_the_gpu():
    from fast_sp_gs_amd import lib
    L = lib.load()
    rc = L.fsgs_knn_topk(10, 5, 3, 64, None, None, None, None, None)
    assert rc != 0 and b"knn_topk" in L.fsgs_last_error()
    rc = L.fsgs_sh_encode_forward(8, 3, 9, None, None, None)
    assert rc != 0
    R = ctypes.c_int64(-1)
    assert L.fsgs_gs_prepare_scan(0, None, None, None, 0, ctypes.addressof(R), None) == 0 and R.value == 0


def test_renderer_wrapper_is_importable_and_binds_by_name():
    from fast_sp_gs_amd.renderer import gs_2d_render as m
    from fast_sp_gs_amd._C import get_C_function
    assert m._GS_2D_Render._render_forward is get_C_function('GS_2D_render_forward')
    assert m.GS_prepare is get_C_function('GS_prepare')


def test_operator_signatures_match_the_reference_prototypes():
    """Positional arity of every exported operator against the reference's host-function prototypes
    (tests/golden/op_signatures.json, written by tests/golden/make_op_signatures.py from the `m.def` bindings and the
    C++ definitions): the reference's bindings are positional (no py::arg except cdist_top), so a drop-in must take the
    same number of leading parameters in the same order; parameters added here must come after them and have defaults."""
    import inspect
    import json
    from fast_sp_gs_amd._C import _ops
    table = json.loads((ROOT / "tests" / "golden" / "op_signatures.json").read_text())
    on_path = REFERENCE_NAMES + [
        'gs_2d_fast_preprocess_forward', 'gs_2d_fast_preprocess_backward', 'gs_2d_fast_compute_transmat_forward',
        'gs_2d_fast_compute_trans_mat_backward', 'GS_2D_fast_render_forward', 'GS_2D_fast_render_backward',
        'gs_2d_topk_weights', 'fusedssim', 'fusedssim_backward', 'simple_knn', 'gs_preprocess_forward',
        'gs_preprocess_backward', 'gaussian_rasterize_forward', 'gaussian_rasterize_backward', 'gaussian_topk_weights',
        'gaussian_rasterize_extra_forward', 'gaussian_rasterize_extra_backward', 'gs_compute_cov3D_forward',
        'gs_compute_cov3D_backward', 'gs_compute_cov2D_forward', 'gs_compute_cov2D_backward']
    checked = 0
    for name, entry in table.items():
        fn = getattr(_ops, name, None)
        if fn is None:
            assert name not in on_path, f"{name} is on the path but not exported"
            continue
        ref = entry['params']
        mine = [p for p in inspect.signature(fn).parameters.values()
                if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
        assert len(mine) >= len(ref), (name, len(mine), len(ref))
        for p in mine[len(ref):]:
            assert p.default is not inspect.Parameter.empty, (name, p.name, "added parameter without a default")
        for p, r in zip(mine, ref):
            # what the reference lets a caller leave out (None for an optional tensor, a bound default) must be
            # acceptable here too: a default here, if any, is None / the same kind of value
            if r['optional'] and p.default is not inspect.Parameter.empty:
                assert p.default is None, (name, p.name)
        # same names where the reference spells them correctly (e.g. it has 'sh_featrues', 'tiles_touch')
        same = sum(p.name == r['name'] for p, r in zip(mine, ref))
        assert same >= len(ref) - 3, (name, [(p.name, r['name']) for p, r in zip(mine, ref) if p.name != r['name']])
        checked += 1
    assert checked >= 37
    for name in on_path:
        assert name in table and hasattr(_ops, name), name
