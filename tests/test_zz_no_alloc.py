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
_WARM = [False]


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
    if not _WARM[0]:    # the first call on a device looks the array's address up; what is measured is every later one
        warm = torch.empty(n * REC, dtype=torch.uint8, device=DEV)
        _abi.grad_stats_mt_static(table.ptr, n, code, bpc, warm.data_ptr(), False, stream)
        _WARM[0] = True
    torch.cuda.synchronize()
    # the driver's own count of free device memory (torch's allocator statistics would not see a hipMalloc
    # made inside the library) and torch's, before the call and right after it, before anything is freed
    free_before, _ = torch.cuda.mem_get_info()
    torch_before = torch.cuda.memory_allocated()
    _abi.grad_stats_mt_static(table.ptr, n, code, bpc, got.data_ptr(), False, stream)
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before and torch.cuda.memory_allocated() == torch_before
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
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


def test_static_variant_inside_a_captured_graph():
    """After one eager call on the device, the entry point can be recorded into a HIP graph (it
    allocates nothing and looks nothing up any more): three replays over changing gradients, with eager
    work and synchronisations between them, each equal to elx_grad_stats_mt on the same gradients."""
    torch.cuda.set_device(0)
    code, bpc = _abi.ELX_F16, 16
    sizes = [200_000, 70_001, 4096]
    grads = _grads(sizes, code, seed=21)
    table = _table(grads, sizes)
    n = len(sizes)
    got = torch.zeros(n * REC, dtype=torch.uint8, device=DEV)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _abi.grad_stats_mt_static(table.ptr, n, code, bpc, got.data_ptr(), False, side.cuda_stream)    # eager, first
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side, capture_error_mode='thread_local'):
        _abi.grad_stats_mt_static(table.ptr, n, code, bpc, got.data_ptr(), False, torch.cuda.current_stream().cuda_stream)
    partials = torch.empty(n * bpc * REC, dtype=torch.uint8, device=DEV)
    want = torch.zeros(n * REC, dtype=torch.uint8, device=DEV)
    for replay in range(3):
        for i, g in enumerate(grads):    # the program's own eager work between the replays: new gradients
            g.mul_(1.5)
            if replay == 1 and i == 1:
                g[77] = float('nan')
        torch.cuda.synchronize()
        got.fill_(0xCD)
        graph.replay()
        torch.cuda.synchronize()
        _abi.grad_stats_mt(table.ptr, n, code, bpc, partials.data_ptr(), want.data_ptr(), False,
                           torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        a, b = want.cpu().numpy().view(_abi.STATS_DTYPE), got.cpu().numpy().view(_abi.STATS_DTYPE)
        assert a.tobytes() == b.tobytes(), replay
        assert list(a['overflow']) == [0, 1 if replay >= 1 else 0, 0]


_FIRST_CALL_UNDER_CAPTURE = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
from elixir_amd import _abi
from elixir_amd.chunk import DeviceTable
torch.cuda.set_device(0)
g = torch.ones(4096, dtype=torch.float16, device='cuda')
rows = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
rows[0]['grad'], rows[0]['n_alloc'], rows[0]['n_valid'] = g.data_ptr(), 4096, 4096
table = DeviceTable(rows, torch.device('cuda', 0))
out = torch.zeros(16, dtype=torch.uint8, device='cuda')
side = torch.cuda.Stream()
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
code = None
with torch.cuda.graph(graph, stream=side, capture_error_mode='thread_local'):
    try:
        _abi.grad_stats_mt_static(table.ptr, 1, _abi.ELX_F16, 1, out.data_ptr(), False, torch.cuda.current_stream().cuda_stream)
    except _abi.ElxError as e:
        code = e.code
assert code == _abi.ELX_E_STATE, code
# outside capture the same call goes through, and from then on it may be captured
_abi.grad_stats_mt_static(table.ptr, 1, _abi.ELX_F16, 1, out.data_ptr(), False, torch.cuda.current_stream().cuda_stream)
torch.cuda.synchronize()
rec = out.cpu().numpy().view(_abi.STATS_DTYPE)[0]
assert rec['sumsq'] == 4096.0 and rec['overflow'] == 0, rec
print('refused under capture, accepted afterwards')
"""


def test_first_call_on_a_device_under_capture_is_refused(tmp_path):
    """The first call on a device has to look the array's address up, which is not something to do while a
    stream captures: it is refused with ELX_E_STATE before anything is launched (in a process of its own:
    in this one the address is known already)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_path / 'first_call.py'
    script.write_text(_FIRST_CALL_UNDER_CAPTURE)
    proc = subprocess.run([sys.executable, str(script), root], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stdout
    assert 'refused under capture, accepted afterwards' in proc.stdout
