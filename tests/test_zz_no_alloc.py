"""elx_grad_stats_mt_static -- the entry point that takes no workspace and allocates nothing -- against
elx_grad_stats_mt on the same tables, straight through the C ABI: identical ElxStats records (same
kernels, same reduction order), on two calls in a row of which the second is smaller (the fixed
partials array still holds the first call's records), and the size limit is refused with ELX_E_SIZE."""
import numpy as np
import pytest
import torch

from elixir_amd import _abi
from elixir_amd.chunk import DeviceTable

pytestmark = pytest.mark.gpu
DEV = 'cuda'
REC = _abi.STATS_DTYPE.itemsize
TORCH = {_abi.ELX_F16: torch.float16, _abi.ELX_BF16: torch.bfloat16, _abi.ELX_F32: torch.float32}


def _grads(sizes, code, seed, poison=None):
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    out = []
    for i, n in enumerate(sizes):
        g = (torch.randn(n, device=DEV, generator=gen) * 3.0).to(TORCH[code])
        if poison is not None and i == poison[0]:
            g[poison[1]] = float('inf')
        out.append(g)
    return out


def _table(grads, valid):
    rows = np.zeros(len(grads), dtype=_abi.CHUNK_DTYPE)
    for i, (g, nv) in enumerate(zip(grads, valid)):
        rows[i]['grad'] = g.data_ptr()
        rows[i]['n_alloc'] = g.numel()
        rows[i]['n_valid'] = nv
    return DeviceTable(rows, torch.device(DEV, 0))


def _both(table, n, code, bpc):
    """(records of elx_grad_stats_mt with a caller workspace, records of the static variant)."""
    stream = torch.cuda.current_stream().cuda_stream
    partials = torch.empty(n * bpc * REC, dtype=torch.uint8, device=DEV)
    want = torch.full((n * REC, ), 0xAB, dtype=torch.uint8, device=DEV)
    got = torch.full((n * REC, ), 0xCD, dtype=torch.uint8, device=DEV)
    _abi.grad_stats_mt(table.ptr, n, code, bpc, partials.data_ptr(), want.data_ptr(), False, stream)
    before = torch.cuda.memory_allocated()
    _abi.grad_stats_mt_static(table.ptr, n, code, bpc, got.data_ptr(), False, stream)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return want.cpu().numpy().view(_abi.STATS_DTYPE), got.cpu().numpy().view(_abi.STATS_DTYPE)


@pytest.mark.parametrize('code', [_abi.ELX_F16, _abi.ELX_BF16, _abi.ELX_F32])
def test_static_partials_match_the_workspace_variant_twice(code):
    torch.cuda.set_device(0)
    # first call: five chunks, ragged valid heads, an inf in chunk 3; 64 workgroups per chunk
    sizes = [1 << 20, (1 << 20) + 8, 300_001, 1 << 19, 4096]
    valid = [1 << 20, 1 << 20, 299_999, (1 << 19) - 7, 0]
    grads = _grads(sizes, code, seed=11, poison=(3, 12345))
    table = _table(grads, valid)
    want, got = _both(table, len(sizes), code, 64)
    assert want.tobytes() == got.tobytes()
    assert list(want['overflow']) == [0, 0, 0, 1, 0]
    ref = [float((g[:nv].double()**2).sum()) for g, nv in zip(grads, valid)]
    for i in (0, 1, 2, 4):
        assert abs(want['sumsq'][i] - ref[i]) <= 1e-6 * ref[i] + 0.0

    # second call, smaller: two chunks, seven workgroups each, no overflow -- the array still holds the
    # first call's 320 partials (one of them flagged) and none of them may leak into these records
    sizes2 = [70_000, 33_333]
    grads2 = _grads(sizes2, code, seed=12)
    table2 = _table(grads2, sizes2)
    want2, got2 = _both(table2, 2, code, 7)
    assert want2.tobytes() == got2.tobytes()
    assert list(want2['overflow']) == [0, 0]
    for i in range(2):
        ref2 = float((grads2[i].double()**2).sum())
        assert abs(got2['sumsq'][i] - ref2) <= 1e-6 * ref2


def test_static_partials_refuse_what_does_not_fit():
    torch.cuda.set_device(0)
    cap = _abi.static_partials()
    assert cap == 65536
    n = cap // 1024 + 1    # 65 chunks x 1024 workgroups: one row too many
    g = torch.zeros(256, dtype=torch.float16, device=DEV)
    table = _table([g] * n, [256] * n)
    out = torch.zeros(n * REC, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(_abi.ElxError) as e:
        _abi.grad_stats_mt_static(table.ptr, n, _abi.ELX_F16, 1024, out.data_ptr(), False, stream)
    assert e.value.code == _abi.ELX_E_SIZE
    # the largest launch that fits goes through
    _abi.grad_stats_mt_static(table.ptr, n - 1, _abi.ELX_F16, 1024, out.data_ptr(), False, stream)
    torch.cuda.synchronize()
    rec = out.cpu().numpy().view(_abi.STATS_DTYPE)
    assert not rec['overflow'].any() and not rec['sumsq'].any()
