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


def _job(kind, c, rows, H=1, W=1, k=1, stride=1, pad=0, x=256, C=512):
    j = _hip.FactorJob()
    j.kind, j.c, j.rows, j.H, j.W = kind, c, rows, H, W
    j.kh = j.kw = k
    j.sh = j.sw = stride
    j.ph = j.pw = pad
    j.dh = j.dw = 1
    j.alpha, j.x, j.C = 1., x, C
    return j


def test_grouped_factor_plan_needs_no_device():
    """The plan of a grouped call (scratch, executed flops) is host arithmetic; bad lists are
    refused before anything is launched."""
    lib = _hip.load()
    jobs = [_job(_hip.FACTOR_LINEAR, 784, 128, C=1 << 20),
            _job(_hip.FACTOR_CONV_G, 64, 32, 56, 56, C=2 << 20),          # long reduction: k-splits
            _job(_hip.FACTOR_CONV_A, 64, 32, 56, 56, k=3, pad=1, C=3 << 20),   # correlation kernels
            _job(_hip.FACTOR_CONV_A, 128, 32, 28, 28, k=3, stride=2, pad=1, C=4 << 20)]
    arr = (_hip.FactorJob * len(jobs))(*jobs)
    assert lib.kfac_factor_grouped_workspace_bytes(len(jobs), arr) > 64 * 64 * 4
    # executed flops: the same tiles and reduction chunks as the single-product plans
    single = (lib.kfac_factor_executed_flops(784, 128) + lib.kfac_factor_executed_flops(64, 32 * 56 * 56)
              + lib.kfac_factor_conv_a_executed_flops(32, 64, 56, 56, 3, 3, 1, 1, 1, 1, 1, 1, 0)
              + lib.kfac_factor_conv_a_executed_flops(32, 128, 28, 28, 3, 3, 2, 2, 1, 1, 1, 1, 0))
    assert abs(lib.kfac_factor_grouped_executed_flops(len(jobs), arr) - single) <= 1e-9 * single
    assert lib.kfac_factor_grouped(0, None, None, 0, None) == 0
    assert lib.kfac_factor_grouped(1, None, None, 0, None) == 1
    assert lib.kfac_factor_grouped(len(jobs), arr, None, 0, None) == 2            # no scratch
    bad = (_hip.FactorJob * 1)(_job(7, 4, 4))
    assert lib.kfac_factor_grouped(1, bad, None, 0, None) == 1                    # unknown kind
    twice = (_hip.FactorJob * 2)(_job(_hip.FACTOR_LINEAR, 4, 4), _job(_hip.FACTOR_LINEAR, 4, 4))
    assert lib.kfac_factor_grouped(2, twice, None, 0, None) == 1                  # one output twice
