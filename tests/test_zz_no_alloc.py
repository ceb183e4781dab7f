"""The entry point that allocates nothing, kfac_damped_inverse_batched_static (its scratch
is an array inside the library), against kfac_damped_inverse_batched with a caller-provided
workspace: same kernels, same launch sequence, so the results must agree bit for bit.  Two
calls in a row, the second on a smaller list (the array then still holds the first call's
contents), with all tensors allocated before the calls."""
import ctypes

import pytest
import torch

from torchsso import _hip

pytestmark = pytest.mark.gpu


def _spd(n, gen, dev):
    m = torch.randn(n, n + 8, generator=gen)
    return (m @ m.t() / (n + 8)).to(dev).contiguous()


def _call_pair(lib, mats, damps, dev):
    """(workspace entry point, static entry point) results for one list, through the C ABI."""
    count = len(mats)
    dims = _hip.int_array([m.shape[0] for m in mats])
    damp = _hip.f32_array(damps)
    src = _hip.ptr_array(mats, 'matrix')
    stream = _hip.stream_ptr(dev)
    want = [torch.full_like(m, float('nan')) for m in mats]
    got = [torch.full_like(m, float('nan')) for m in mats]
    info_w = torch.full((count,), -1, dtype=torch.int32, device=dev)
    info_g = torch.full((count,), -1, dtype=torch.int32, device=dev)
    need = lib.kfac_inverse_workspace_bytes(count, dims)
    assert need <= lib.kfac_static_workspace_bytes()
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)['allocation.all.allocated']
    st = lib.kfac_damped_inverse_batched_static(count, dims, src, damp, _hip.ptr_array(got, 'out'),
                                                info_g.data_ptr(), stream)
    assert st == 0
    # nothing went through torch's allocator during the call (hipMalloc inside the library
    # would not show here; the library has none: the scratch is a __device__ array)
    assert torch.cuda.memory_stats(dev)['allocation.all.allocated'] == before
    st = lib.kfac_damped_inverse_batched(count, dims, src, damp, _hip.ptr_array(want, 'out'),
                                         info_w.data_ptr(), ws.data_ptr(), need, stream)
    assert st == 0
    torch.cuda.synchronize()
    return want, got, info_w, info_g


def test_static_scratch_inverse_equals_workspace_inverse_twice_in_a_row():
    lib = _hip.load()
    dev = torch.device('cuda:0')
    gen = torch.Generator().manual_seed(7)
    first = [_spd(n, gen, dev) for n in (700, 129, 384, 64, 1)]
    second = [_spd(n, gen, dev) for n in (200, 33)]          # smaller: stale scratch behind it
    for mats in (first, second):
        damps = [1e-3 * (i + 1) for i in range(len(mats))]
        want, got, info_w, info_g = _call_pair(lib, mats, damps, dev)
        assert info_w.tolist() == [0] * len(mats) and info_g.tolist() == [0] * len(mats)
        for m, d, w, g in zip(mats, damps, want, got):
            assert torch.equal(w, g), 'n = %d: static-scratch result differs' % m.shape[0]
            # and it is the inverse: float64 on the device, bar 1e-4 relative Frobenius
            ref = torch.linalg.inv(m.double() + d * torch.eye(m.shape[0], dtype=torch.float64,
                                                              device=dev))
            err = ((g.double() - ref).norm() / ref.norm()).item()
            assert err < 1e-4, (m.shape[0], err)


def test_static_scratch_calls_on_two_streams_are_put_in_order():
    """Two calls on two streams share the one array: the library makes the second wait for
    the first (an event per device), so both give the bits of the workspace entry point."""
    lib = _hip.load()
    dev = torch.device('cuda:0')
    gen = torch.Generator().manual_seed(11)
    lists = [[_spd(n, gen, dev) for n in (900, 130)], [_spd(n, gen, dev) for n in (640, 257, 5)]]
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    keep, got, want = [], [], []
    torch.cuda.synchronize()
    for rep in range(3):
        for mats, st in zip(lists, streams):
            dims = _hip.int_array([m.shape[0] for m in mats])
            damp = _hip.f32_array([1e-3] * len(mats))
            outs = [torch.full_like(m, float('nan')) for m in mats]
            info = torch.full((len(mats),), -1, dtype=torch.int32, device=dev)
            src, dst = _hip.ptr_array(mats, 'matrix'), _hip.ptr_array(outs, 'out')
            keep.append((dims, damp, src, dst, info))
            # (the tensors were made on the default stream, idle since the synchronisation)
            assert lib.kfac_damped_inverse_batched_static(len(mats), dims, src, damp, dst,
                                                          info.data_ptr(), st.cuda_stream) == 0
            got.append(outs)
    torch.cuda.synchronize()
    for mats in lists:
        dims = _hip.int_array([m.shape[0] for m in mats])
        damp = _hip.f32_array([1e-3] * len(mats))
        outs = [torch.empty_like(m) for m in mats]
        info = torch.zeros(len(mats), dtype=torch.int32, device=dev)
        need = lib.kfac_inverse_workspace_bytes(len(mats), dims)
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        assert lib.kfac_damped_inverse_batched(len(mats), dims, _hip.ptr_array(mats, 'matrix'), damp,
                                               _hip.ptr_array(outs, 'out'), info.data_ptr(),
                                               ws.data_ptr(), need, _hip.stream_ptr(dev)) == 0
        want.append(outs)
    torch.cuda.synchronize()
    for i, outs in enumerate(got):
        for w, g in zip(want[i % 2], outs):
            assert torch.equal(w, g), 'call %d on stream %d differs' % (i, i % 2)


def test_static_scratch_rejects_what_does_not_fit():
    lib = _hip.load()
    dev = torch.device('cuda:0')
    n = 1500                                                  # 9 MB of scratch > 8 MiB
    m = torch.eye(n, device=dev)
    out = torch.zeros_like(m)
    info = torch.zeros(1, dtype=torch.int32, device=dev)
    st = lib.kfac_damped_inverse_batched_static(1, _hip.int_array([n]), _hip.ptr_array([m]), None,
                                                _hip.ptr_array([out]), info.data_ptr(),
                                                _hip.stream_ptr(dev))
    assert st == 4
    torch.cuda.synchronize()
    assert out.abs().sum().item() == 0                        # nothing was launched
    with pytest.raises(_hip.KfacHipError, match='too large'):
        _hip.check(st, 'kfac_damped_inverse_batched_static')
