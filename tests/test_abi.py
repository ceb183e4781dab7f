"""The C-ABI library: it loads without a GPU, exports every function that
include/kfac_hip.h declares, the ctypes binding covers exactly those, and the
argument checks that need no device reject bad input with an error code."""
import ctypes
import os
import re

import pytest

from torchsso import _hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'kfac_hip.h')


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(kfac_[a-z0-9_]+)\s*\(', text)))


def test_library_is_built_and_loads():
    assert os.path.exists(_hip.lib_path()), 'run python pytorch-sso_amd/build_ext.py'
    lib = _hip.load()
    assert lib.kfac_abi_version() == 2


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 15
    raw = ctypes.CDLL(_hip.lib_path())
    for n in names:
        assert hasattr(raw, n), 'header declares %s but the library does not export it' % n
    assert sorted(_hip.signatures()) == names


def test_header_cites_the_reference_for_each_entry_point():
    text = open(HEADER).read()
    for n in declared_functions():
        if n.endswith(('_workspace_bytes', '_executed_flops')) or n == 'kfac_abi_version':
            continue
        idx = text.index(n + '(')
        comment = text[:idx].rsplit('/*', 1)[1]
        flat = ' '.join(comment.replace('*', ' ').split())
        if 'no counterpart in the reference' in flat:
            # says so instead of citing, and names the callers it exists for
            assert 'cannot allocate' in flat
            continue
        assert re.search(r'\.py:\d+', comment), '%s: no reference file:line in its comment' % n


def test_workspace_queries_need_no_device():
    lib = _hip.load()
    assert lib.kfac_factor_workspace_bytes(4608, 1568) >= 0
    assert lib.kfac_factor_workspace_bytes(64, 401408) > 0          # split-k partials
    dims = _hip.int_array([100, 300])
    assert lib.kfac_inverse_workspace_bytes(2, dims) >= 4 * (100 * 100 + 300 * 300)
    assert lib.kfac_precondition_workspace_bytes(1, _hip.int_array([10]), _hip.int_array([20])) >= 800
    assert lib.kfac_vector_workspace_bytes(3) > 0


def test_argument_errors_are_codes_not_crashes():
    lib = _hip.load()
    # null pointers / bad sizes are rejected before anything touches a device
    assert lib.kfac_factor_linear(None, 8, 4, 4, 1, 1.0, 0.0, None, None, None, 0, None) == 1
    assert lib.kfac_factor_conv_g(None, 1, 1, 1, 1, 1.0, 0.0, None, None, None, 0, None) == 1
    assert lib.kfac_rowsq_sum(None, 1, 1, 1, None, None, None, None) == 1
    assert lib.kfac_bn_diag_cov(None, 1, 1, 1, None, 1.0, None, None, None, 0, None) == 1
    assert lib.kfac_bn_diag_cov_workspace_bytes(32, 64) == 32 * 64 * 4
    assert lib.kfac_bn_diag_cov_workspace_bytes(0, 64) == 0
    # the entry point with built-in scratch refuses what does not fit it, before any launch
    assert lib.kfac_static_workspace_bytes() == 8 << 20
    big = _hip.int_array([2000])
    one = (ctypes.c_void_p * 1)(1 << 20)
    two = (ctypes.c_void_p * 1)(2 << 20)
    assert lib.kfac_inverse_workspace_bytes(1, big) > lib.kfac_static_workspace_bytes()
    assert lib.kfac_damped_inverse_batched_static(1, big, one, None, two, one, None) == 4
    assert lib.kfac_damped_inverse_batched_static(1, big, one, None, one, one, None) == 1
    with pytest.raises(_hip.KfacHipError):
        _hip.check(2, 'x')
