#!/usr/bin/env python3
"""Writes tests/golden/step_cases.npz: small seeded inputs and the outputs PyTorch's CPU ops give
for them.  The reference's own Adam (ColossalAI) is not available offline, and the parity target
names torch.optim.Adam / AdamW on CPU as the semantics, so the expected values come from there:

    flag    = isinf(g).any() | isnan(g).any()                 (elixir/chunk/core/chunk.py:214-216)
    l2      = g.float().norm(2).item() ** 2                     (chunk.py:218-221)
    g32     = g.float().div_(div_scale)                         (the inner optimizer's div_scale)
    p, m, v = torch.optim.Adam / AdamW (foreach=False) on CPU
    lowp    = p.to(float16 | bfloat16)                          (chunk.py:414)
    scale   = torch._amp_update_scale_ trajectories (the dynamic scaler with hysteresis 1)

Run from the repository root:  python tests/golden/make_golden.py
Needs only torch and numpy.  The file it writes is committed; tests never regenerate it.
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, 'step_cases.npz')

LOWP = {'f16': torch.float16, 'bf16': torch.bfloat16, 'f32': torch.float32}

# name, dtype, n, adamw, weight_decay, betas, div_scale, steps
CASES = [
    ('f32_adam', 'f32', 389, False, 0.0, (0.9, 0.999), -1.0, 3),
    ('f32_adamw', 'f32', 131, True, 0.01, (0.9, 0.999), -1.0, 2),
    ('f32_l2', 'f32', 131, False, 0.01, (0.9, 0.999), -1.0, 2),
    ('f16_scale64', 'f16', 389, True, 0.0, (0.9, 0.999), 64.0, 3),
    ('f16_scale65536_wd', 'f16', 263, True, 0.1, (0.9, 0.999), 65536.0, 2),
    ('f16_clip_scale', 'f16', 263, True, 0.1, (0.9, 0.999), 5379818.327114731, 2),
    ('bf16_adamw', 'bf16', 389, True, 0.01, (0.9, 0.999), -1.0, 2),
    ('bf16_clip_scale', 'bf16', 263, True, 0.01, (0.9, 0.95), 20.34274291050705, 2),
    ('f16_low_beta1', 'f16', 131, True, 0.05, (0.4, 0.9), 8.0, 2),
    ('f16_l2', 'f16', 131, False, 0.05, (0.9, 0.999), 8.0, 2),
]


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def main():
    out = {}
    gen = torch.Generator().manual_seed(20240531)
    names = []
    for name, dt, n, adamw, wd, betas, div_scale, steps in CASES:
        lowp = LOWP[dt]
        scale = div_scale if div_scale > 0 else 1.0
        p0 = torch.randn(n, generator=gen) * 0.02
        m0 = torch.randn(n, generator=gen) * 1e-4
        v0 = torch.rand(n, generator=gen) * 1e-6
        param = torch.nn.Parameter(p0.clone())
        cls = torch.optim.AdamW if adamw else torch.optim.Adam
        opt = cls([param], lr=1e-3, betas=betas, eps=1e-8, weight_decay=wd, foreach=False)
        st = opt.state[param]
        st['step'] = torch.tensor(0.0)
        st['exp_avg'] = m0.clone()
        st['exp_avg_sq'] = v0.clone()
        out[f'{name}/p_init'], out[f'{name}/m_init'], out[f'{name}/v_init'] = p0.numpy(), m0.numpy(), v0.numpy()
        for s in range(steps):
            g = (torch.randn(n, generator=gen) * (1e-3 * scale)).to(lowp)
            g32 = g.float()
            if div_scale > 0:
                g32.div_(div_scale)
            param.grad = g32
            opt.step()
            out[f'{name}/g{s}'] = bits(g)
            out[f'{name}/p_out{s}'] = param.data.numpy().copy()
            out[f'{name}/m_out{s}'] = st['exp_avg'].numpy().copy()
            out[f'{name}/v_out{s}'] = st['exp_avg_sq'].numpy().copy()
            out[f'{name}/lowp{s}'] = bits(param.data.to(lowp))
            out[f'{name}/l2_{s}'] = np.array(g.float().norm(2).item()**2, dtype=np.float64)
        out[f'{name}/meta'] = np.array([n, int(adamw), wd, betas[0], betas[1], div_scale, steps], dtype=np.float64)
        names.append(f'{name}:{dt}')
    out['case_names'] = np.array(names)

    # overflow flags on crafted inputs
    for dt in ('f16', 'bf16', 'f32'):
        lowp = LOWP[dt]
        base = (torch.randn(300, generator=gen) * 10).to(lowp)
        variants = {'clean': base.clone()}
        for label, val, pos in (('pinf_first', float('inf'), 0), ('ninf_last', float('-inf'), 299),
                                ('nan_mid', float('nan'), 150)):
            t = base.clone()
            t[pos] = val
            variants[label] = t
        big = base.clone()
        big[7] = torch.finfo(lowp).max
        big[8] = -torch.finfo(lowp).max
        variants['largest_finite'] = big
        for label, t in variants.items():
            flag = bool(torch.isinf(t).any().item() | torch.isnan(t).any().item())
            out[f'overflow/{dt}/{label}/g'] = bits(t)
            out[f'overflow/{dt}/{label}/flag'] = np.array(flag)

    # low-precision rounding of special fp32 values
    special = np.array([0x00000000, 0x80000000, 0x33000000, 0x33000001, 0x337FFFFF, 0x33800000, 0x387FC000, 0x387FE000,
                        0x38800000, 0x477FE000, 0x477FEFFF, 0x477FF000, 0x47800000, 0x7F7FFFFF, 0x7F800000, 0xFF800000,
                        0x3F801000, 0x3F803000, 0x3F808000, 0x3F818000, 0x3F800000, 0x3F807FFF, 0x00000001, 0x007FFFFF,
                        0x00800000, 0x3EAAAAAB, 0xC2F6E979], dtype=np.uint32)
    rnd = torch.randint(0, 2**31 - 1, (1500, ), generator=gen).numpy().astype(np.uint32) * 2 + 1
    vals = np.concatenate([special, rnd]).view(np.float32)
    vals = vals[~np.isnan(vals)]
    out['cast/x'] = vals
    out['cast/f16'] = bits(torch.from_numpy(vals.copy()).to(torch.float16))
    out['cast/bf16'] = bits(torch.from_numpy(vals.copy()).to(torch.bfloat16))

    # loss-scale trajectories from torch's own scale update (hysteresis 1 semantics)
    patterns = {
        'clean_growth': [0] * 7,
        'one_overflow': [0, 0, 1, 0, 0, 0, 0, 0],
        'burst': [1, 1, 1, 0, 0, 0, 1, 0, 0, 0, 0, 0],
        'alternating': [0, 1, 0, 1, 0, 0, 0, 1, 0, 0, 0],
    }
    for label, seq in patterns.items():
        scale = torch.tensor([1024.0])
        growth = torch.tensor([0], dtype=torch.int32)
        traj = []
        for found in seq:
            torch._amp_update_scale_(scale, growth, torch.tensor([float(found)]), 2.0, 0.5, 3)
            traj.append(float(scale.item()))
        out[f'scaler/{label}/found'] = np.array(seq, dtype=np.int32)
        out[f'scaler/{label}/scale'] = np.array(traj, dtype=np.float64)

    # gradient landing with torch's CPU ops: the payload divided in place by a power-of-two group
    # size (chunk.py:299; for a power of two the division is the multiplication by the reciprocal
    # that the device kernel performs), copied into a shard of the chunk's type (chunk.py:314), and
    # the flags of what then sits in the shard (chunk.py:214-221)
    lgen = torch.Generator().manual_seed(777)
    lowps = {'f16': torch.float16, 'bf16': torch.bfloat16}
    for dt, tdt in (('f16', torch.float16), ('bf16', torch.bfloat16), ('f32', torch.float32)):
        for label, spread in (('tame', 1.0), ('wild', 6.0)):
            x = (torch.randn(3000, generator=lgen) * torch.exp(torch.randn(3000, generator=lgen) * spread)).to(tdt)
            out[f'land/{dt}/{label}/x'] = bits(x)
            for pg in (1, 4):
                y = x.clone()
                if pg > 1:
                    y /= pg
                targets = {dt: y} if tdt != torch.float32 else {'f32': y, **{k: y.to(v) for k, v in lowps.items()}}
                for tname, shard in targets.items():
                    key = f'land/{dt}/{label}/pg{pg}/{tname}'
                    out[key] = bits(shard)
                    bad = bool(torch.isinf(shard).any() | torch.isnan(shard).any())
                    out[key + '/flag'] = np.array(bad)
                    if not bad:
                        out[key + '/l2'] = np.array(shard.float().norm(2).item()**2, dtype=np.float64)

    np.savez_compressed(OUT, **out)
    print(f'wrote {OUT}: {len(out)} arrays, {os.path.getsize(OUT)} bytes')


if __name__ == '__main__':
    main()
