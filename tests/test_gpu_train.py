"""End-to-end: a small network trained through ElixirModule + ElixirOptimizer(HybridAdam) against
plain PyTorch training of an identical copy -- the shape of the reference's own tests
(test/wrapper/test_optimizer.py: fp32, rtol 2e-6 / atol 2e-5 on the weights after the step;
test/wrapper/test_amp.py: fp16 against master-weight AMP, assert_close defaults)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

import elixir_amd as ea
from elixir_amd import _abi

pytestmark = pytest.mark.gpu
DEV = 'cuda'


class Net(nn.Module):
    """Dense layers only: no scatter-add in backward, so two runs of the same step produce the
    same gradients bit for bit and the comparison sees the optimizers, not atomics."""

    def __init__(self, width=24, hidden=32):
        super().__init__()
        self.inp = nn.Linear(width, hidden)
        self.norm1 = nn.LayerNorm(hidden)
        self.fc1 = nn.Linear(hidden, 4 * hidden)
        self.fc2 = nn.Linear(4 * hidden, hidden)
        self.norm2 = nn.LayerNorm(hidden)
        self.head = nn.Linear(hidden, 50, bias=False)

    def forward(self, x):
        h = self.inp(x.to(self.inp.weight.dtype))
        h = h + self.fc2(torch.nn.functional.gelu(self.fc1(self.norm1(h))))
        return self.head(self.norm2(h)).float().logsumexp(-1).mean()


def batch(gen):
    return torch.randn(8, 16, 24, device=DEV, generator=gen)


def groups_of(model, wd):
    decay = [p for p in model.parameters() if p.dim() > 1]
    exempt = [p for p in model.parameters() if p.dim() == 1]
    return [dict(params=decay, weight_decay=wd), dict(params=exempt, weight_decay=0.0)]


def wrap(model, dtype, chunk_size=4096, **kw):
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    module = ea.ElixirModule(model, ea.greedy_search(named, chunk_size, dtype), dtype=dtype)
    inner = ea.HybridAdam(groups_of(model, 0.1), lr=1e-2, weight_decay=0.1)
    return module, ea.ElixirOptimizer(module, inner, **kw)


def test_fp32_training_matches_torch_adamw():
    torch.manual_seed(0)
    ref = Net().to(DEV)
    model = copy.deepcopy(ref)
    ropt = torch.optim.AdamW(groups_of(ref, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, torch.float32)
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(4):
        x = batch(gen)
        ropt.zero_grad()
        ref(x).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        module.materialize_params()
        sd = module.state_dict()
        for name, want in ref.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'step {step} {name}')


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
def test_frozen_parameters_stay_out_of_the_chunks(dtype):
    """Parameters that need no gradient (module.py:83-90, optimizer.py:248-249): they are moved to the
    training dtype and the GPU and otherwise left alone -- no chunk holds them, the optimizer has no
    range for them, ``state_dict`` hands them out and ``load_state_dict`` takes them back -- while the
    rest trains as torch's AdamW trains it with the same parameters frozen."""
    torch.manual_seed(0)
    ref = Net().to(DEV)
    for p in (ref.norm1.weight, ref.norm1.bias, ref.fc2.bias):
        p.requires_grad_(False)
    model = copy.deepcopy(ref)
    frozen = {'norm1.weight', 'norm1.bias', 'fc2.bias'}
    trainable = [(n, p) for n, p in model.named_parameters() if p.requires_grad]
    assert {n for n, p in model.named_parameters() if not p.requires_grad} == frozen
    ropt = torch.optim.AdamW([dict(params=[p for p in ref.parameters() if p.requires_grad and p.dim() > 1], weight_decay=0.1),
                              dict(params=[p for p in ref.parameters() if p.requires_grad and p.dim() == 1], weight_decay=0.0)],
                             lr=1e-2)
    module = ea.ElixirModule(model, ea.greedy_search([(n, p.numel()) for n, p in trainable], 4096, dtype), dtype=dtype)
    # the groups name every parameter, frozen ones too: the wrapper drops those (optimizer.py:248-249)
    inner = ea.HybridAdam(groups_of(model, 0.1), lr=1e-2, weight_decay=0.1)
    opt = ea.ElixirOptimizer(module, inner, initial_scale=64.0)
    assert set(module.no_grad_state_dict) == frozen and not frozen & set(module.grad_state_dict)
    assert sum(len(g['params']) for g in opt.param_groups) == len(trainable)
    for name in frozen:
        t = module.no_grad_state_dict[name]
        assert t.dtype == dtype and t.is_cuda and not t.requires_grad
    chunked = {t for c in module.param_chunks for t in c.tensors_info}
    assert not any(module.no_grad_state_dict[n] in chunked for n in frozen)
    before = {n: module.no_grad_state_dict[n].clone() for n in frozen}
    initial = {n: t.detach().float().cpu().clone() for n, t in ref.state_dict().items()}
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(3):
        x = batch(gen)
        ropt.zero_grad()
        ref(x).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        assert opt.last_step_info['found_inf'] is False
    module.materialize_params()
    sd = module.state_dict()
    for name, want in ref.state_dict().items():
        if name in frozen:
            assert torch.equal(sd[name], before[name]) and sd[name].dtype == dtype
            assert torch.equal(sd[name].float().cpu(), want.to(dtype).float().cpu())
        elif dtype == torch.float32:
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'{name}')
        else:
            # (fp16 gradients are other gradients: after three steps of Adam only the size of the move is comparable)
            moved = (sd[name].float() - initial[name]).abs().max().item()
            assert 0 < moved <= 3 * 1e-2 * 1.2 and torch.isfinite(sd[name]).all(), (name, moved)
    # loading a state dict writes the frozen ones where they live
    new = {n: (t.float() + 1.0) for n, t in sd.items()}
    module.load_state_dict(new)
    for name in frozen:
        assert torch.equal(module.no_grad_state_dict[name].float().cpu(), (before[name].float() + 1.0).to(dtype).float().cpu())


class TiedNet(nn.Module):
    """The output projection shares its weight with the embedding, as GPT-2's does."""

    def __init__(self, vocab=50, hidden=32):
        super().__init__()
        self.emb = nn.Embedding(vocab, hidden)
        self.fc = nn.Linear(hidden, hidden)
        self.head = nn.Linear(hidden, vocab, bias=False)
        self.head.weight = self.emb.weight

    def forward(self, idx):
        return self.head(torch.tanh(self.fc(self.emb(idx)))).float().logsumexp(-1).mean()


@pytest.mark.parametrize('chunk_size', [1600, 4096])
def test_a_tied_weight_lands_once_and_trains_like_torch(chunk_size):
    """One parameter under two names (``emb.weight`` / ``head.weight``): it sits in one chunk once -- alone in
    it with the smaller chunk size, as the reference's searches place a parameter that is used twice
    (search/simple.py:33) --, its gradient (the sum over both uses) lands once from the hook of backward, and
    ``state_dict`` hands the trained values out under both names."""
    torch.manual_seed(0)
    ref = TiedNet().to(DEV)
    model = copy.deepcopy(ref)
    assert model.head.weight is model.emb.weight
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    assert [n for n, _ in named] == ['emb.weight', 'fc.weight', 'fc.bias']
    ropt = torch.optim.AdamW(ref.parameters(), lr=1e-2, weight_decay=0.1)
    module = ea.ElixirModule(model, ea.greedy_search(named, chunk_size, torch.float32), dtype=torch.float32)
    opt = ea.ElixirOptimizer(module, ea.HybridAdam(model.parameters(), lr=1e-2, weight_decay=0.1))
    assert [c.num_tensors for c in module.param_chunks] == ([1, 2] if chunk_size == 1600 else [3])
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(3):
        idx = torch.randint(0, 50, (8, 16), device=DEV, generator=gen)
        ropt.zero_grad()
        ref(idx).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(idx))
        opt.step()
        assert opt.last_step_info['found_inf'] is False
    module.materialize_params()
    assert model.head.weight is model.emb.weight
    sd = module.state_dict()
    assert torch.equal(sd['head.weight'], sd['emb.weight'])
    for name, want in ref.state_dict().items():
        torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=name)
    module.load_state_dict({n: t + 1.0 for n, t in sd.items()})
    again = module.state_dict()
    for name in sd:
        assert torch.equal(again[name], sd[name] + 1.0), name


def test_two_wrapped_models_in_one_process_do_not_disturb_each_other():
    """Two modules with an optimizer each (fp16 with a dynamic loss scale, bf16 with a constant one, other
    chunk sizes, both clipped) share one GPU: its record arena, the library's tables and streams.  Stepped in
    turns they end with the bits they end with when one trains after the other."""

    def run(in_turns):
        torch.manual_seed(0)
        a, b = Net().to(DEV), Net(hidden=48).to(DEV)
        ma, oa = wrap(a, torch.float16, chunk_size=4096, initial_scale=64.0, max_norm=1.0)
        mb, ob = wrap(b, torch.bfloat16, chunk_size=16384, max_norm=0.5)
        ga, gb = torch.Generator(device=DEV).manual_seed(1), torch.Generator(device=DEV).manual_seed(2)

        def step(m, o, g):
            o.zero_grad()
            o.backward(m(batch(g)))
            o.step()

        if in_turns:
            for _ in range(4):
                step(ma, oa, ga)
                step(mb, ob, gb)
        else:
            for _ in range(4):
                step(ma, oa, ga)
            for _ in range(4):
                step(mb, ob, gb)
        return [c.paired_chunk.shard.clone() for m in (ma, mb) for c in m.param_chunks] + \
               [t.clone() for o in (oa, ob) for c in o._binding.chunks for t in o._binding.moments(c)]

    for u, v in zip(run(True), run(False)):
        assert torch.equal(u, v)


class NetWithBuffers(nn.Module):
    """Batch normalisation brings buffers along: two floating-point ones and an integer count per layer (the
    reference's own optimizer test trains a ResNet, test/wrapper/test_optimizer.py:55)."""

    def __init__(self, width=24, hidden=32):
        super().__init__()
        self.inp = nn.Linear(width, hidden, bias=False)
        self.bn1 = nn.BatchNorm1d(hidden)
        self.fc = nn.Linear(hidden, hidden, bias=False)
        self.bn2 = nn.BatchNorm1d(hidden)
        self.head = nn.Linear(hidden, 10)

    def forward(self, x):
        h = torch.relu(self.bn1(self.inp(x.to(self.inp.weight.dtype))))
        h = torch.relu(self.bn2(self.fc(h)))
        return self.head(h).float().logsumexp(-1).mean()


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
def test_buffers_move_with_the_module_and_stay_out_of_the_chunks(dtype):
    """module.py:91-95: floating-point buffers go to the training dtype and the GPU, integer ones keep their
    type; no chunk holds them, ``state_dict`` hands them out as the wrapped module keeps them.  In fp32 the
    whole state after three steps, running statistics included, is the one plain PyTorch training reaches."""
    torch.manual_seed(0)
    ref = NetWithBuffers().to(DEV)
    model = copy.deepcopy(ref)
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    buffers = {n for n, _ in model.named_buffers()}
    assert len(buffers) == 6
    ropt = torch.optim.AdamW(groups_of(ref, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, dtype, chunk_size=1024, initial_scale=64.0)
    for name, buf in model.named_buffers():
        assert buf.is_cuda and buf.dtype == (torch.int64 if name.endswith('num_batches_tracked') else dtype), name
    assert sum(c.num_tensors for c in module.param_chunks) == len(named)
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(3):
        x = torch.randn(64, 24, device=DEV, generator=gen)
        ropt.zero_grad()
        ref(x).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        assert opt.last_step_info['found_inf'] is False
    module.materialize_params()
    sd = module.state_dict()
    assert set(sd) == set(ref.state_dict())
    for name, want in ref.state_dict().items():
        if name.endswith('num_batches_tracked'):
            assert sd[name].dtype == torch.int64 and int(sd[name]) == 3
        elif dtype == torch.float32:
            torch.testing.assert_close(sd[name].cpu(), want.cpu(), rtol=2e-6, atol=2e-5, msg=name)
        else:
            assert sd[name].dtype == (dtype if name in buffers else torch.float32) and torch.isfinite(sd[name].float()).all()


class NetWithEmptyParameters(nn.Module):
    """Two parameters without elements, one of them first in the module's own order."""

    def __init__(self, width=24, hidden=32):
        super().__init__()
        self.nothing = nn.Parameter(torch.zeros(0))
        self.inp = nn.Linear(width, hidden)
        self.norm = nn.LayerNorm(hidden)
        self.none_either = nn.Parameter(torch.zeros(0, 3))
        self.head = nn.Linear(hidden, 50, bias=False)

    def forward(self, x):
        h = self.norm(torch.tanh(self.inp(x.to(self.inp.weight.dtype))))
        return self.head(h).float().logsumexp(-1).mean() + self.nothing.sum() + self.none_either.sum()


def test_parameters_without_elements_are_carried_along():
    """A parameter of zero elements sits in a chunk with an empty range (chunk.py:223-247), gets no fake
    parameter (optimizer.py:251-253: ``begin >= end``), lands nothing and comes back from ``state_dict``;
    the rest trains as under torch's AdamW."""
    torch.manual_seed(0)
    ref = NetWithEmptyParameters().to(DEV)
    model = copy.deepcopy(ref)
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    assert named[0] == ('nothing', 0) and ('none_either', 0) in named
    ropt = torch.optim.AdamW(groups_of(ref, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, torch.float32)
    assert sum(len(g['params']) for g in opt.param_groups) == len(named) - 2
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(3):
        x = batch(gen)
        ropt.zero_grad()
        ref(x).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
    module.materialize_params()
    sd = module.state_dict()
    for name, want in ref.state_dict().items():
        assert sd[name].shape == want.shape
        torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=name)


@pytest.mark.parametrize('make', [lambda ps: torch.optim.SGD(ps, lr=5e-2, momentum=0.9, nesterov=True),
                                  lambda ps: torch.optim.RMSprop(ps, lr=1e-3)], ids=['sgd', 'rmsprop'])
def test_inner_optimizer_outside_the_fused_list_runs_unfused(make):
    """optimizer.py:54-56,211-214: any element-wise torch optimizer may sit inside the wrapper as long
    as nothing has to be unscaled (fp32, no clipping); it then steps on views of the chunk storage.
    Same optimizer on an identical plain copy: the same weights, to the reference's own tolerance."""
    torch.manual_seed(0)
    ref = Net().to(DEV)
    model = copy.deepcopy(ref)
    ropt = make(list(ref.parameters()))
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    module = ea.ElixirModule(model, ea.greedy_search(named, 4096, torch.float32), dtype=torch.float32)
    opt = ea.ElixirOptimizer(module, make(list(model.parameters())))
    assert not opt.scaled_optimizer and opt.loss_scale == 1.0
    gen = torch.Generator(device=DEV).manual_seed(1)
    for step in range(4):
        x = batch(gen)
        ropt.zero_grad()
        ref(x).backward()
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        assert opt.last_step_info['found_inf'] is False and opt.last_step_info['combined_scale'] == -1
        module.materialize_params()
        sd = module.state_dict()
        for name, want in ref.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'step {step} {name}')
    # with clipping such an optimizer cannot be used: nothing would apply the coefficient
    torch.manual_seed(0)
    model = Net().to(DEV)
    module = ea.ElixirModule(model, ea.greedy_search(named, 4096, torch.float32), dtype=torch.float32)
    opt = ea.ElixirOptimizer(module, make(list(model.parameters())), max_norm=1e-3)
    opt.zero_grad()
    opt.backward(module(batch(gen)))
    with pytest.raises(AssertionError):
        opt.step()


def test_fp16_training_matches_master_weight_amp_and_recovers_from_overflow():
    torch.manual_seed(0)
    master = Net().to(DEV)                         # fp32 master copy trained by plain torch
    model = copy.deepcopy(master)
    ropt = torch.optim.AdamW(groups_of(master, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, torch.float16, initial_scale=1024.0, hysteresis=1, growth_interval=1000)
    gen = torch.Generator(device=DEV).manual_seed(2)
    scale = 1024.0
    for step in range(5):
        x = batch(gen)
        poison = step == 2
        # reference side: fp16 working copy of the fp32 master, scaled loss, unscale in fp32
        work = copy.deepcopy(master).half()
        (work(x) * scale).backward()
        grads = [p.grad for p in work.parameters()]
        if poison:
            grads[3].view(-1)[5] = float('inf')
        if any((~torch.isfinite(g)).any() for g in grads):
            scale *= 0.5
        else:
            for p, g in zip(master.parameters(), grads):
                p.grad = g.float() / scale
            ropt.step()
        # this build
        assert opt.loss_scale == (1024.0 if step <= 2 else 512.0)
        opt.zero_grad()
        opt.backward(module(x))
        if poison:
            pc = module.param_chunks[0]
            pc.shard[7] = float('inf')
            pc.invalidate_stats()    # the shard changed behind the chunk's back: flags from the landing are stale
        opt.step()
        assert opt.last_step_info['found_inf'] == poison
        module.materialize_params()
        sd = module.state_dict()
        for name, want in master.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), msg=f'step {step} {name}')
        # the parameters the forward pass sees are the rounded masters
        for name, p in model.named_parameters():
            assert torch.equal(p.data.cpu(), sd[name].half())
    assert opt.loss_scale == scale == 512.0


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_low_precision_training_is_bit_identical_to_a_master_weight_loop_with_the_same_optimizer(dtype):
    """The shape of the reference's own test/wrapper/test_amp.py: the same optimizer on both sides, so
    that the comparison pins the plumbing (packing, ranges, landing from hooks, unscale, writeback,
    what the next forward pass sees) -- here to the bit: HybridAdam standing alone on an fp32 master
    copy, fed the low-precision gradients of a rounded working copy and the loss scale as divisor."""
    torch.manual_seed(0)
    master = Net().to(DEV)
    model = copy.deepcopy(master)
    sopt = ea.HybridAdam(groups_of(master, 0.1), lr=1e-2, weight_decay=0.1)
    scale = 256.0 if dtype == torch.float16 else 1.0
    kw = dict(initial_scale=scale, hysteresis=1, growth_interval=1000) if dtype == torch.float16 else {}
    module, opt = wrap(model, dtype, **kw)
    gen = torch.Generator(device=DEV).manual_seed(2)
    for step in range(5):
        x = batch(gen)
        work = copy.deepcopy(master).to(dtype)
        (work(x) * scale).backward()
        for p, w in zip(master.parameters(), work.parameters()):
            p.grad_dtype = None    # an fp32 parameter carrying a low-precision gradient
            p.grad = w.grad
        sopt.step(div_scale=scale if scale != 1.0 else -1)
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        assert opt.last_step_info['found_inf'] is False and opt.loss_scale == scale
        module.materialize_params()
        sd = module.state_dict()
        for name, want in master.state_dict().items():
            assert torch.equal(sd[name], want.cpu()), f'step {step} {name}'
        for (name, p), w in zip(model.named_parameters(), master.parameters()):
            assert torch.equal(p.data, w.data.to(dtype)), f'step {step} {name}: what the forward pass sees'


def test_forward_after_a_step_sees_the_new_weights_without_being_told():
    """The reference's forward pass gathers its chunks anew after every step; here the module's
    parameters are private copies of the shards, refreshed by the first forward pass after a step.
    A loop that never calls materialize_params must train exactly like one that does."""
    torch.manual_seed(0)
    base = Net().to(DEV)
    runs = []
    for explicit in (True, False):
        model = copy.deepcopy(base)
        module, opt = wrap(model, torch.float16, initial_scale=256.0, hysteresis=1)
        gen = torch.Generator(device=DEV).manual_seed(7)
        losses = []
        for step in range(4):
            loss = module(batch(gen))
            losses.append(float(loss.detach()))
            opt.zero_grad()
            opt.backward(loss)
            opt.step()
            if explicit:
                module.materialize_params()
        runs.append((losses, {k: v.clone() for k, v in module.state_dict().items()}))
    assert runs[0][0] == runs[1][0] and runs[0][0][0] != runs[0][0][-1]
    for name, want in runs[0][1].items():
        assert torch.equal(runs[1][1][name], want), name


def test_state_dict_round_trip_and_load():
    torch.manual_seed(3)
    model = Net().to(DEV)
    module, opt = wrap(model, torch.bfloat16)
    sd = module.state_dict()
    new = {k: torch.randn_like(v) for k, v in sd.items()}
    module.load_state_dict(new)
    back = module.state_dict()
    for k in new:
        assert torch.equal(back[k], new[k])
        assert torch.equal(module.state_dict(from_param=True)[k], new[k].bfloat16())


def test_resume_from_checkpoint_is_bit_identical():
    """Train, save weights + optimizer state + scaler, go on; a fresh module and optimizer that load
    the checkpoint and see the same batches end with the same bits.  The save point sits right after
    a skipped step with hysteresis 2, so the scaler's counters matter."""
    torch.manual_seed(3)
    base = Net().to(DEV)

    def run(model, steps, gen, opt_pair=None, poison_at=()):
        module, opt = opt_pair or wrap(model, torch.float16, initial_scale=512.0, hysteresis=2, growth_interval=3)
        for step in steps:
            x = batch(gen)
            opt.zero_grad()
            opt.backward(module(x))
            if step in poison_at:
                pc = module.param_chunks[-1]
                pc.shard[pc.n_valid - 1] = float('-inf')
                pc.invalidate_stats()
            opt.step()
            module.materialize_params()
        return module, opt

    gen = torch.Generator(device=DEV).manual_seed(9)
    module, opt = run(copy.deepcopy(base), range(0, 4), gen, poison_at=(3,))
    assert opt.last_step_info['found_inf'] is True and opt.loss_scale == 1024.0    # grew at step 3 (0-2 clean), armed, not backed off
    weights = module.state_dict()
    ckpt = opt.state_dict()
    gen_state = gen.get_state()
    # the saved moments are copies: going on must not change them
    frozen = {i: st['exp_avg'].clone() for i, st in ckpt['state'].items()}
    module, opt = run(None, range(4, 9), gen, opt_pair=(module, opt), poison_at=(5,))
    assert all(torch.equal(frozen[i], st['exp_avg']) for i, st in ckpt['state'].items())
    # 3: armed; 4: clean; 5: second overflow of the window -> 512; 6-8: three clean steps -> 1024 again
    assert opt.loss_scale == 1024.0 and opt.grad_scaler._growth_step == 0

    gen2 = torch.Generator(device=DEV).manual_seed(0)
    gen2.set_state(gen_state)
    fresh_module, fresh_opt = wrap(copy.deepcopy(base), torch.float16, initial_scale=2.0, hysteresis=1)
    fresh_module.load_state_dict(weights)
    fresh_opt.load_state_dict(ckpt)
    assert fresh_opt.loss_scale == 1024.0
    fresh_module, fresh_opt = run(None, range(4, 9), gen2, opt_pair=(fresh_module, fresh_opt), poison_at=(5,))

    assert fresh_opt.loss_scale == opt.loss_scale == 1024.0
    for a, b in zip(module.param_chunks, fresh_module.param_chunks):
        assert torch.equal(a.paired_chunk.shard, b.paired_chunk.shard) and torch.equal(a.shard, b.shard)
        for x, y in zip(opt._binding.moments(a.paired_chunk), fresh_opt._binding.moments(b.paired_chunk)):
            assert torch.equal(x, y)
    sa, sb = opt.state_dict(), fresh_opt.state_dict()
    assert [st['step'] for st in sa['state'].values()] == [st['step'] for st in sb['state'].values()] == [7] * len(
        sa['state'])
    assert sa['grad_scaler']['growth_step'] == sb['grad_scaler']['growth_step']
    assert sa['grad_scaler']['hysteresis_step'] == sb['grad_scaler']['hysteresis_step']


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_clipped_training_matches_torchs_clip_grad_norm(dtype):
    """Global L2 clipping end to end: the combined scale of optimizer.py:166-183 against
    ``torch.nn.utils.clip_grad_norm_`` (coefficient max_norm / (norm + 1e-6), applied only above the
    threshold) followed by torch's AdamW on fp32 master weights.  max_norm is small enough that
    every step clips."""
    torch.manual_seed(1)
    master = Net().to(DEV)
    model = copy.deepcopy(master)
    ropt = torch.optim.AdamW(groups_of(master, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, dtype, max_norm=0.05)
    gen = torch.Generator(device=DEV).manual_seed(4)
    for step in range(4):
        x = batch(gen)
        if dtype == torch.float32:
            work = master
            ropt.zero_grad()
            work(x).backward()
        else:
            work = copy.deepcopy(master).to(dtype)
            work(x).backward()
            for p, w in zip(master.parameters(), work.parameters()):
                p.grad = w.grad.float()
        norm = torch.nn.utils.clip_grad_norm_(master.parameters(), 0.05)
        assert float(norm) > 0.05
        ropt.step()
        opt.zero_grad()
        opt.backward(module(x))
        opt.step()
        info = opt.last_step_info
        assert info['found_inf'] is False
        assert abs(info['total_norm'] - float(norm)) <= 2e-6 * float(norm)
        assert info['combined_scale'] > 1.0
        module.materialize_params()
        sd = module.state_dict()
        for name, want in master.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'step {step} {name}')


def test_chunks_land_from_hooks_during_backward(monkeypatch):
    """module.py:177-190: a chunk lands as soon as its last gradient exists -- one launch per chunk,
    issued from inside backward, gradients freed right away -- and the shards hold exactly what a
    landing after backward would have put there."""
    import elixir_amd.module as M
    torch.manual_seed(5)
    model = Net().to(DEV)
    module, opt = wrap(model, torch.float16, initial_scale=256.0)
    n_chunks = len(module.param_chunks)
    assert n_chunks >= 4
    calls = []
    inside = {'flag': False}
    real = M.land_tensors

    def spy(chunks, grad_of, mul=1.0):
        calls.append((len(chunks), inside['flag'], sum(p.grad is not None for p in model.parameters())))
        return real(chunks, grad_of, mul)

    monkeypatch.setattr(M, 'land_tensors', spy)
    real_backward = torch.Tensor.backward

    def marked_backward(self, *a, **k):
        inside['flag'] = True
        try:
            return real_backward(self, *a, **k)
        finally:
            inside['flag'] = False

    monkeypatch.setattr(torch.Tensor, 'backward', marked_backward)
    gen = torch.Generator(device=DEV).manual_seed(6)
    x = batch(gen)
    opt.zero_grad()
    opt.backward(module(x))
    assert len(calls) == n_chunks and all(n == 1 and was_inside for n, was_inside, _ in calls)
    n_params = sum(1 for _ in model.parameters())
    assert max(alive for _, _, alive in calls) < n_params        # earlier chunks had already freed theirs
    assert all(p.grad is None for p in model.parameters())
    assert all(pc._stats_pending for pc in module.param_chunks)
    landed = [pc.shard.clone() for pc in module.param_chunks]

    # the same gradients, landed after a plain backward
    monkeypatch.setattr(torch.Tensor, 'backward', real_backward)
    (module(x) * opt.loss_scale).backward()
    for pc in module.param_chunks:
        pc.invalidate_stats()
    module.land_gradients()
    for pc, want in zip(module.param_chunks, landed):
        assert torch.equal(pc.shard.view(torch.int16), want.view(torch.int16))
    module.module.zero_grad(set_to_none=True)
    opt.step()
    assert opt.last_step_info['found_inf'] is False


def test_hook_driven_backward_takes_the_device_decided_step(oracle, monkeypatch):
    """The flow training takes (module.py:177-190, fetcher.py:133-153: a chunk is reduced as soon as it is
    ready; optimizer.py:137-142): ``opt.backward`` lands the chunks from the hooks, one launch per chunk,
    the last chunk first.  The optimizer gave every chunk its record slot in chunk order when it was built,
    so the flags still end up side by side and the step is decided on the device: no stats launch, no host
    read before the update.  Its result has the bits of the host-decided step on the same gradients, and
    of the oracle's step."""
    import elixir_amd.chunk as C
    from helpers import CODE, to_np
    from oracle import oracle as O
    dtype = torch.float16
    torch.manual_seed(11)
    model = Net().to(DEV)
    twin = copy.deepcopy(model)
    module, opt = wrap(model, dtype, initial_scale=256.0, hysteresis=1, max_norm=0.5)
    module_h, opt_h = wrap(twin, dtype, initial_scale=256.0, hysteresis=1, max_norm=0.5)
    opt_h.gated_step = False
    chunks = module.param_chunks
    assert len(chunks) >= 4
    poison = {'on': False}

    def maybe_poison(g):    # an overflow that backward itself produces, so that the landing sees it
        if poison['on']:
            g = g.clone()
            g.view(-1)[3] = float('inf')
        return g

    model.head.weight.register_hook(maybe_poison)
    slots = [c._stats_slot for c in chunks]
    assert slots == list(range(slots[0], slots[0] + len(chunks))) and all(c._stats_pinned for c in chunks)

    order = []
    real_land = C._land_tensors_run

    def spy_land(arena, run, *a, **k):
        order.extend(run)
        return real_land(arena, run, *a, **k)

    monkeypatch.setattr(C, '_land_tensors_run', spy_land)
    stats_launches = []
    for name in ('grad_partials_mt', 'grad_stats_mt', 'grad_stats'):
        real = getattr(_abi, name)
        monkeypatch.setattr(_abi, name, lambda *a, _real=real, _name=name, **k: (stats_launches.append(_name), _real(*a, **k))[1])
    reads = []
    real_read = C.StatsArena.read
    monkeypatch.setattr(C.StatsArena, 'read', lambda self, lo, hi: (reads.append((lo, hi)), real_read(self, lo, hi))[1])

    gen = torch.Generator(device=DEV).manual_seed(12)
    scaler = O.DynamicGradScalerOracle(initial_scale=256.0, min_scale=1, max_scale=2**24, hysteresis=1)
    for step in range(3):
        x = batch(gen)
        order.clear()
        opt.zero_grad()
        poison['on'] = step == 1
        opt.backward(module(x))
        assert [c.chunk_id for c in order[:len(chunks)]] != sorted(c.chunk_id for c in chunks)    # not in chunk order
        assert set(order) == set(chunks) and len(order) == len(chunks)                          # one launch per chunk
        assert [c._stats_slot for c in chunks] == slots                                         # nobody moved
        assert opt._stats_source() == ('arena', slots[0])
        # the oracle's and the host-decided twin's view of the same gradients and state
        ochunks = []
        for pc in chunks:
            fc = pc.paired_chunk
            m, v = opt._binding.moments(fc)
            segs = []
            for group in opt.param_groups:
                for fake in group['params']:
                    if opt.param_to_optim_chunk[fake] is fc:
                        b, e = opt.param_to_range[fake]
                        segs.append(O.OracleSegment(b, e, lr=group['lr'], betas=tuple(group['betas']), eps=group['eps'],
                                                    weight_decay=group['weight_decay'],
                                                    bias_correction=group['bias_correction'],
                                                    step=opt.state[fake]['step'] if opt.state[fake] else 0))
            segs.sort(key=lambda sg: sg.begin)
            ochunks.append(O.OracleChunk(lowp=to_np(pc.shard), master=to_np(fc.shard), m=to_np(m), v=to_np(v),
                                         valid_end=pc.n_valid, segments=segs))
        for pc, ph in zip(chunks, module_h.param_chunks):
            ph.shard.copy_(pc.shard)
            ph.invalidate_stats()
        opt_h.mark_gradients_scaled()

        stats_launches.clear()
        reads.clear()
        opt.step()
        assert stats_launches == [] and reads == []      # the flags never left the device before the update
        opt_h.step()
        info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=0.5)
        assert opt.last_step_info['found_inf'] == opt_h.last_step_info['found_inf'] == info['found_inf'] == (step == 1)
        assert opt.loss_scale == opt_h.loss_scale == info['loss_scale']
        if step != 1:
            assert opt.last_step_info['combined_scale'] == opt_h.last_step_info['combined_scale']
            assert opt.last_step_info['total_norm'] == opt_h.last_step_info['total_norm']
            assert abs(opt.last_step_info['combined_scale'] - info['combined_scale']) <= 1e-6 * info['combined_scale']
        for pc, ph, oc in zip(chunks, module_h.param_chunks, ochunks):
            ma, va = opt._binding.moments(pc.paired_chunk)
            mb, vb = opt_h._binding.moments(ph.paired_chunk)
            for a, b in ((pc.shard, ph.shard), (pc.paired_chunk.shard, ph.paired_chunk.shard), (ma, mb), (va, vb)):
                assert torch.equal(a.view(torch.int16) if a.dtype == dtype else a.view(torch.int32),
                                   b.view(torch.int16) if b.dtype == dtype else b.view(torch.int32)), step
            assert_close = np.testing.assert_allclose
            assert_close(to_np(pc.paired_chunk.shard), oc.master, rtol=1e-6, atol=1e-9)
            assert_close(to_np(ma), oc.m, rtol=1e-6, atol=1e-8)
            assert_close(to_np(va), oc.v, rtol=1e-6, atol=1e-10)
        module_h.mark_params_stale()
    assert [st['step'] for st in opt.state.values()] == [st['step'] for st in opt_h.state.values()]
    assert set(st['step'] for st in opt.state.values()) == {2}


def test_backward_by_grad_lands_like_backward():
    """optimizer.py:230-236: a pipeline stage that is not the last receives the (already scaled) gradient
    of its output and runs backward from there.  The same gradients reach the shards as through
    ``backward`` on a loss built from that output, the gradients count as scaled, and the step that follows
    has the same bits."""
    torch.manual_seed(21)
    model = Net().to(DEV)
    twin = copy.deepcopy(model)
    module, opt = wrap(model, torch.float16, initial_scale=128.0, hysteresis=1)
    module2, opt2 = wrap(twin, torch.float16, initial_scale=128.0, hysteresis=1)
    gen = torch.Generator(device=DEV).manual_seed(22)
    x = batch(gen)
    upstream = torch.tensor(3.0, device=DEV)    # d(total loss) / d(this stage's output), loss scale not included
    opt.zero_grad()
    out = module(x)
    opt.backward_by_grad(out, upstream * opt.loss_scale)
    opt2.zero_grad()
    opt2.backward(module2(x) * upstream)
    assert opt.optim_state == opt2.optim_state == ea.OptimState.SCALED
    for a, b in zip(module.param_chunks, module2.param_chunks):
        assert a._stats_pending and torch.equal(a.shard.view(torch.int16), b.shard.view(torch.int16))
    assert all(p.grad is None for p in model.parameters())
    opt.step()
    opt2.step()
    assert opt.last_step_info['found_inf'] is False and opt.last_step_info == opt2.last_step_info
    for a, b in zip(module.param_chunks, module2.param_chunks):
        assert torch.equal(a.paired_chunk.shard, b.paired_chunk.shard)
        assert torch.equal(a.shard.view(torch.int16), b.shard.view(torch.int16))


def test_tables_prepared_at_backward_follow_late_hyperparameter_changes():
    """``backward`` prepares the tables of the coming step ahead of time; a learning rate changed
    between backward and step must still be the one the step uses."""
    torch.manual_seed(2)
    ref = Net().to(DEV)
    model = copy.deepcopy(ref)
    ropt = torch.optim.AdamW(groups_of(ref, 0.1), lr=1e-2, weight_decay=0.1)
    module, opt = wrap(model, torch.float32)
    gen = torch.Generator(device=DEV).manual_seed(8)
    for step in range(4):
        x = batch(gen)
        ropt.zero_grad()
        ref(x).backward()
        opt.zero_grad()
        opt.backward(module(x))
        assert opt.optim._prepared is not None                 # built ahead of the step
        ahead = opt.optim._prepared
        if step % 2 == 1:                                      # a scheduler that fires late
            for g in list(ropt.param_groups) + list(opt.param_groups):
                g['lr'] = g['lr'] * 0.5
        ropt.step()
        opt.step()
        assert opt.optim._prepared is None                     # consumed
        module.materialize_params()
        sd = module.state_dict()
        for name, want in ref.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'step {step} {name}')
        del ahead


def test_fine_tune_loop_of_the_reference_with_torch_adam_and_a_warmup_schedule():
    """The shape of example/fine-tune/elixir_mini.py:70-110 and func_module.py:46-66: an fp32 module, a plain
    ``torch.optim.Adam`` with a decay group and a no-decay group as the inner optimizer,
    ``ElixirOptimizer(model, optimizer, init_step=True)``, a linear warm-up / decay schedule built ON THE
    WRAPPER, and the loop zero_grad -> forward -> optimizer.backward -> optimizer.step -> lr_scheduler.step.
    Against the same loop on a plain copy (which takes the allocation step's zero-gradient update by hand):
    the same weights to the reference's own tolerance, the same learning rates."""

    def schedule(opt, warm=3, total=10):    # transformers' get_linear_schedule_with_warmup
        return torch.optim.lr_scheduler.LambdaLR(
            opt, lambda s: s / max(1, warm) if s < warm else max(0.0, (total - s) / max(1, total - warm)))

    def groups(model):
        decay = [p for n, p in model.named_parameters() if 'norm' not in n and 'bias' not in n]
        rest = [p for n, p in model.named_parameters() if 'norm' in n or 'bias' in n]
        return [dict(params=decay, weight_decay=0.01), dict(params=rest, weight_decay=0.0)]

    torch.manual_seed(0)
    ref = Net().to(DEV)
    model = copy.deepcopy(ref)
    gen = torch.Generator(device=DEV).manual_seed(1)
    x0 = batch(gen)
    # What init_step does (optimizer.py:94-113): one step with zero gradients, at the constructor's
    # learning rate, on the master weights only -- the parameters the first forward pass sees are not
    # refreshed (optimizer.py:113 passes update_flag=False).  On the plain copy: take the first batch's
    # gradients on the untouched weights, then the zero-gradient step, then the first real step.
    ropt = torch.optim.Adam(groups(ref), lr=2e-3, eps=1e-8)
    ref(x0).backward()
    first_grads = [p.grad.clone() for p in ref.parameters()]
    for p in ref.parameters():
        p.grad = torch.zeros_like(p)
    ropt.step()
    rsched = schedule(ropt)

    optimizer = torch.optim.Adam(groups(model), lr=2e-3, eps=1e-8)
    named = [(n, p.numel()) for n, p in model.named_parameters()]
    module = ea.ElixirModule(model, ea.greedy_search(named, 4096, torch.float32), None, dtype=torch.float32,
                             use_fused_kernels=True)
    optimizer = ea.ElixirOptimizer(module, optimizer, init_step=True)
    assert isinstance(optimizer, torch.optim.Optimizer) and not optimizer.scaled_optimizer
    lr_scheduler = schedule(optimizer)

    for step in range(6):
        x = x0 if step == 0 else batch(gen)
        if step == 0:
            for p, g in zip(ref.parameters(), first_grads):
                p.grad = g
        else:
            ropt.zero_grad()
            ref(x).backward()
        ropt.step()
        rsched.step()

        optimizer.zero_grad()
        loss = module(x)
        optimizer.backward(loss)
        optimizer.step()
        lr_scheduler.step()

        assert [g['lr'] for g in optimizer.param_groups] == [g['lr'] for g in ropt.param_groups]
        module.materialize_params()
        sd = module.state_dict()
        for name, want in ref.state_dict().items():
            torch.testing.assert_close(sd[name], want.cpu(), rtol=2e-6, atol=2e-5, msg=f'step {step} {name}')
    assert lr_scheduler.last_epoch == 6 and optimizer.param_groups[0]['lr'] == pytest.approx(2e-3 * 4 / 7)
