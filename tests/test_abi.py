"""The C ABI as a loadable artefact: every symbol that include/fm_hip.h declares is exported by
libfmhip.so with the arity the ctypes binding uses, and argument validation -- which runs
before any HIP call -- reports errors through fm_last_error(). No kernel is launched here.
"""

import ctypes
import os
import re

import pytest

from forgeminds_amd.kernels import _hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fm_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|size_t|const char\*)\s+(fm_[a-z_0-9]+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        decls[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return decls


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_hip.LIB_PATH):
        from forgeminds_amd import build
        build.build(verbose=False)
        _hip.reset_for_tests()
    return _hip.lib()


def test_header_and_binding_agree(lib):
    decl = _declared()
    assert len(decl) == 42
    assert set(decl) == set(_hip.SIGNATURES), set(decl) ^ set(_hip.SIGNATURES)
    for name, nargs in decl.items():
        assert hasattr(lib, name), f"{name} is declared in fm_hip.h but not exported"
        assert len(_hip.SIGNATURES[name][1]) == nargs, name


def test_version_and_error_channel(lib):
    assert lib.fm_version() == 1
    assert lib.fm_set_param(b"no_such_knob", 1) == 1
    assert b"unknown parameter" in lib.fm_last_error()
    assert lib.fm_set_param(b"vocab_threads", 0) == 0
    assert lib.fm_set_param(b"route_presort", 1) == 1      # switches between code paths are not parameters


def test_argument_validation_happens_before_any_launch(lib):
    # bad dtype / shape / k: status FM_ERR_INVALID (1) and a message; nothing touches a GPU
    assert lib.fm_rmsnorm_fwd(None, None, None, None, 4, 8, 7, 0, 1e-6, None) == 1
    assert b"x_dtype" in lib.fm_last_error()
    assert lib.fm_rmsnorm_fwd(None, None, None, None, 4, 0, 2, 2, 1e-6, None) == 1
    assert lib.fm_rmsnorm_fwd(None, None, None, None, 4, 8, 0, 2, 1e-6, None) == 1   # fp32 x, bf16 w
    assert lib.fm_topk(None, None, None, 4, 8, 9, 0, 32, None) == 1
    assert b"selected index k out of range" in lib.fm_last_error()
    assert lib.fm_topk(None, None, None, 4, 8, 2, 0, 16, None) == 1
    assert lib.fm_topk(None, None, None, 4, 4096, 600, 0, 32, None) == 2             # k > 512
    assert lib.fm_kl_fwd(None, None, None, None, None, None, 4, 8, 2, 1.0, 9, None) == 1
    assert lib.fm_ce_fwd(None, None, None, None, None, None, 4, 8, 2, -100, 0, None) == 1
    assert lib.fm_route(None, None, None, None, None, None, None, None, 0, 4, 8, 9, 0, None) == 1
    assert lib.fm_route(None, None, None, None, None, None, None, None, 0, 4, 1024, 2, 0, None) == 2
    # empty problems are a no-op that succeeds
    assert lib.fm_rmsnorm_fwd(None, None, None, None, 0, 8, 2, 2, 1e-6, None) == 0
    assert lib.fm_softmax_fwd(None, None, 0, 8, 2, None) == 0
    assert lib.fm_softmax_bwd(None, None, None, 0, 8, 2, None) == 0
    assert lib.fm_softmax_bwd(None, None, None, 4, 0, 2, None) == 1
    # the one-launch distillation step validates like its parts
    args = (None,) * 10
    assert lib.fm_kl_loss_grad_topk(*args, 4, 8, 9, 2, 32, 1.0, 2, None) == 1          # k > v
    assert lib.fm_kl_loss_grad_topk(*args, 4, 8, 2, 2, 32, 1.0, 0, None) == 1          # reduction none
    assert b"sum or mean" in lib.fm_last_error()
    assert lib.fm_kl_loss_grad_topk(*args, 4, 8, 2, 2, 32, 1.0, 2, None) == 1          # no gradient buffer
    assert lib.fm_rmsnorm_bwd_workspace(0, 8, 2) == 0
    # the router's backward validates like the router
    assert lib.fm_route_bwd(None, None, None, None, None, None, None, 4, 8, 9, 0, None) == 1      # k > e
    assert lib.fm_route_bwd(None, None, None, None, None, None, None, 4, 1024, 2, 0, None) == 2   # e > 512
    assert lib.fm_route_bwd(None, None, None, None, None, None, None, 0, 8, 2, 0, None) == 0      # no rows
    assert lib.fm_route_bwd(None, None, None, None, None, None, None, 4, 8, 2, 0, None) == 1      # NULL buffers


def test_set_param_forgets_cached_workspace_sizes(lib):
    # the sizes follow the launch shapes, which the tuning parameters move
    _hip._WS_BYTES[("probe",)] = 1
    _hip._ROUTE_WS[("probe",)] = 1
    _hip.set_param("norm_bwd_blocks_per_cu", 0)
    assert not _hip._WS_BYTES and not _hip._ROUTE_WS
