"""The entry points enqueue work on the caller's stream and nothing else -- no allocation, no host
synchronisation, no memset node -- so a caller may record them into a HIP graph.  One graph holds a
landing launch, a stats launch, an update launch and the padding refresh; it is replayed several
times with eager work and synchronisations in between, and every replay is compared with the same
launches issued eagerly."""
import numpy as np
import pytest
import torch

from elixir_amd import _abi
from elixir_amd.chunk import DeviceTable
from elixir_amd.hybrid_adam import make_hyper_record
from elixir_amd.launch_plan import FlatBuffer, build_plan

pytestmark = pytest.mark.gpu
DEV = 'cuda'


class _Set:
    """Two flat buffers with a few tensors each, their tables in device memory, and the launches."""

    def __init__(self, seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        self.sizes = [(1 << 16) + 4096, 1 << 15]
        self.valid = [(1 << 16) + 100, (1 << 15) - 777]
        self.payload = [(torch.randn(n, generator=g, device=DEV) * 3.0).half() for n in self.sizes]
        for pl, nv in zip(self.payload, self.valid):
            pl[nv:] = 0
        self.shard = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in self.sizes]
        self.master = [torch.randn(n, generator=g, device=DEV) * 0.02 for n in self.sizes]
        self.m = [torch.randn(n, generator=g, device=DEV) * 1e-3 for n in self.sizes]
        self.v = [torch.rand(n, generator=g, device=DEV) * 1e-5 for n in self.sizes]
        self.state0 = [t.clone() for t in self.master + self.m + self.v]
        hyp = np.concatenate([make_hyper_record(1e-3, 0.9, 0.999, 1e-8, 0.1, 3, True, True),
                              make_hyper_record(1e-3, 0.9, 0.999, 1e-8, 0.0, 3, True, True)])
        bufs = []
        for i, (n, nv) in enumerate(zip(self.sizes, self.valid)):
            cut = nv // 3
            bufs.append(FlatBuffer(grad=self.shard[i].data_ptr(), lowp_out=self.shard[i].data_ptr(),
                                   master=self.master[i].data_ptr(), m=self.m[i].data_ptr(), v=self.v[i].data_ptr(),
                                   n_alloc=n, n_valid=nv, segs=[(0, cut, 0), (cut, nv, 1)]))
        self.plan = build_plan(bufs, 2, 2, len(hyp), _abi.ELX_F16, _abi.ELX_F16)
        self.rows, self.segs = DeviceTable(self.plan.rows, DEV), DeviceTable(self.plan.segs, DEV)
        self.refresh = DeviceTable(self.plan.refresh_rows, DEV) if self.plan.refresh_rows is not None else None
        self.hypers = DeviceTable(hyp, DEV)
        shard_rows = np.zeros(2, dtype=_abi.CHUNK_DTYPE)
        for i in range(2):
            shard_rows[i]['grad'] = self.payload[i].data_ptr()
            shard_rows[i]['lowp_out'] = self.shard[i].data_ptr()
            shard_rows[i]['n_alloc'] = self.sizes[i]
            shard_rows[i]['n_valid'] = self.valid[i]
        self.land_bpr = _abi.check_land_rows(shard_rows, None, _abi.ELX_F16, _abi.ELX_F16)
        self.land_rows = DeviceTable(shard_rows, DEV)
        stat_rows = shard_rows.copy()
        stat_rows['grad'] = stat_rows['lowp_out']
        self.stat_rows = DeviceTable(stat_rows, DEV)
        rec = _abi.STATS_DTYPE.itemsize
        self.land_ws = torch.empty(_abi.land_workspace_records(2, self.land_bpr) * rec, dtype=torch.uint8, device=DEV)
        self.land_out = torch.zeros(2 * rec, dtype=torch.uint8, device=DEV)
        self.stat_bpc = 4
        self.stat_ws = torch.empty(2 * self.stat_bpc * rec, dtype=torch.uint8, device=DEV)
        self.stat_out = torch.zeros(2 * rec, dtype=torch.uint8, device=DEV)

    def launches(self):
        stream = torch.cuda.current_stream().cuda_stream
        _abi.land_grads_mt(self.land_rows.ptr, 2, _abi.ELX_F16, _abi.ELX_F16, 1.0, self.land_bpr, self.land_ws.data_ptr(),
                           self.land_out.data_ptr(), True, stream)
        _abi.grad_stats_mt(self.stat_rows.ptr, 2, _abi.ELX_F16, self.stat_bpc, self.stat_ws.data_ptr(),
                           self.stat_out.data_ptr(), False, stream)
        _abi.adam_step_mt(self.rows.ptr, len(self.plan.rows), self.segs.ptr, len(self.plan.segs), self.hypers.ptr, 2,
                          self.plan.info, 48.0, _abi.ELX_F16, _abi.ELX_F16, 0, stream)
        if self.refresh is not None:
            _abi.writeback_mt(self.refresh.ptr, len(self.plan.refresh_rows), _abi.ELX_F16, self.plan.refresh_max_elems,
                              True, stream)

    def restore(self):
        for t, t0 in zip(self.master + self.m + self.v, self.state0):
            t.copy_(t0)
        for s in self.shard:
            s.fill_(1.0)
        self.land_out.zero_()
        self.stat_out.zero_()

    def snapshot(self):
        return [t.clone() for t in self.master + self.m + self.v + self.shard + [self.land_out, self.stat_out]]


def test_launches_replay_from_a_graph():
    s = _Set(1)
    s.restore()
    s.launches()
    once = s.snapshot()
    s.launches()                       # a second step on the evolved state (the landing re-lands the payload)
    twice = s.snapshot()
    stats = once[-1].cpu().numpy().view(_abi.STATS_DTYPE)
    assert stats['overflow'].tolist() == [0, 0] and np.all(stats['sumsq'] > 0)
    landed = once[-2].cpu().numpy().view(_abi.STATS_DTYPE)    # the landing and the stats pass agree (other summation order)
    assert landed['overflow'].tolist() == [0, 0] and np.allclose(landed['sumsq'], stats['sumsq'], rtol=1e-6, atol=0)

    s.restore()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s.launches()
    torch.cuda.synchronize()

    noise = torch.randn(1 << 20, device=DEV)
    for replay in range(4):
        s.restore()
        noise.mul_(1.0001)                            # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(s.snapshot(), once):
            assert torch.equal(got, want), f'replay {replay}'
        if replay == 2:                               # and once more without restoring: the second step
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip(s.snapshot(), twice):
                assert torch.equal(got, want), 'second step from the graph'
