"""GPU parity at head dims above 128 (the reference pads the head dim to the next power of two,
sb_attn/sb_fwd.py:199, and takes any size that fits its shared memory): bf16 at 256 runs on
matrix-core kernels of its own, bf16 between 129 and 255 rides them zero-padded (float16: tests/test_gpu_float16.py),
fp32 takes the generic kernels.  Same oracle, same tolerances as the other parity tests."""
import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, rel_l2, max_abs, cu_from_lengths, within
from test_gpu_parity import _check_dense, _check_varlen, _ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("T", [1, 33, 64, 127, 128, 129, 200, 512, 1000])
def test_bf16_dense_head_dim_256(T, attend_current):
    _check_dense(2, 3, T, 256, torch.bfloat16, attend_current=attend_current, seed=7 * T + 256, in_scale=0.5)


def test_bf16_head_dims_between_128_and_256_ride_the_256_kernels_zero_padded(monkeypatch):
    _check_dense(1, 2, 150, 160, torch.bfloat16, seed=31, in_scale=0.5)
    _check_dense(2, 2, 300, 192, torch.bfloat16, attend_current=True, seed=32, in_scale=0.5)
    _check_varlen(3, 136, [70, 1, 200, 129], torch.bfloat16, seed=33)
    # and the generic kernels at those head dims stay reachable
    monkeypatch.setenv("SBA_FORCE_GENERIC", "1")
    _check_dense(1, 2, 150, 160, torch.bfloat16, seed=31, in_scale=0.5)
    _check_varlen(2, 256, [130, 45], torch.bfloat16, seed=34)


@pytest.mark.parametrize("attend_current", [False, True])
def test_varlen_head_dim_256(attend_current):
    _check_varlen(3, 256, [300, 1, 129, 700, 64], torch.bfloat16, attend_current=attend_current, seed=35)


def test_unit_variance_inputs_head_dim_256():
    _check_dense(1, 4, 384, 256, torch.bfloat16, seed=36, in_scale=1.0)


@pytest.mark.parametrize("D", [136, 256])
def test_fp32_above_128_takes_the_generic_kernels(D):
    _check_dense(1, 2, 200, D, torch.float32, seed=37 + D)
    _check_varlen(2, D, [130, 45], torch.float32, attend_current=True, seed=38 + D)


def test_many_workgroups_and_long_sweeps_head_dim_256():
    # 6 x 4 x 8 row blocks (every CU busy, sweeps of up to 16 steps, both tile buffers of every kernel in use) against
    # the oracle on the first and the last sequence; all copies of the same sequence must give the same bits
    sb_attn, _ = _ops()
    D, T, rep = 256, 1024, 6
    base = [randn((1, 4, T, D), 240 + i, 0.5, torch.bfloat16) for i in range(3)]
    do = randn((1, 4, T, D), 243, 1.0, torch.bfloat16)
    drem = randn((1, 4, T), 244, 1.0, torch.bfloat16)
    q, k, v = (x.cuda().expand(rep, -1, -1, -1).contiguous().requires_grad_() for x in base)
    o, rem = sb_attn(q, k, v)
    torch.autograd.backward([o, rem], [do.cuda().expand(rep, -1, -1, -1).contiguous(), drem.cuda().expand(rep, -1, -1).contiguous()])
    o_ref, rem_ref, dq, dk, dv = O.sb_attn_grads_oracle(*base, do, drem)
    label = "head_dim 256 H=4 T=1024 (first of 6 copies)"
    within(label, "o", max_abs(o[:1].float().cpu(), o_ref), 2e-2)
    within(label, "rem", max_abs(rem[:1].float().cpu(), rem_ref), 2e-2)
    for name, g, r in (("dq", q.grad, dq), ("dk", k.grad, dk), ("dv", v.grad, dv)):
        within(label, name, rel_l2(g[:1].float().cpu(), r), 5e-2)
        assert torch.equal(g[0], g[rep - 1])
    assert torch.equal(o[0], o[rep - 1]) and torch.equal(rem[0], rem[rep - 1])


def test_recomputing_the_carries_gives_the_same_bits_head_dim_256(monkeypatch):
    sb_attn, sb_attn_varlen = _ops()
    D, lens = 256, [300, 1, 129, 700]
    cu = cu_from_lengths(lens).cuda()
    q, k, v, do = (randn((3, sum(lens), D), 500 + i, 0.5 if i < 3 else 1.0, torch.bfloat16).cuda() for i in range(4))
    drem = randn((3, sum(lens)), 505, 1.0, torch.bfloat16).cuda()

    def packed():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn_varlen(qq, kk, vv, cu, max(lens))
        torch.autograd.backward([o, rem], [do, drem])
        return o, rem, qq.grad, kk.grad, vv.grad

    kept = packed()
    monkeypatch.setenv("SBA_RECOMPUTE_CARRIES", "1")
    for x, y in zip(kept, packed()):
        assert torch.equal(x, y)


def test_seeded_random_sweep_above_128_against_the_oracle():
    # 40 seeded draws: head dims 256 (matrix cores) and 144 / 200 / 224 (zero-padded in bf16, generic in fp32), both
    # masks, dense and packed (with empty documents), lengths at and off the 64 / 128 block edges
    import random
    rng = random.Random(20250311)
    for case in range(40):
        D = rng.choice([256, 256, 256, 144, 200, 224])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.float32])
        ac = rng.random() < 0.3
        seed = rng.randrange(10 ** 6)
        if rng.random() < 0.5:
            B, H = rng.choice([1, 1, 2, 3]), rng.choice([1, 2, 3])
            T = max(1, rng.choice([rng.randrange(1, 70), rng.randrange(1, 400), rng.randrange(1, 1200),
                                   128 * rng.randrange(1, 9), 64 * rng.randrange(1, 17) + rng.choice([-1, 0, 1])]))
            _check_dense(B, H, T, D, dtype, ac, seed=seed, in_scale=0.5, with_drem=rng.random() < 0.8)
        else:
            H = rng.choice([1, 2, 4])
            lens = [max(0 if rng.random() < 0.1 else 1,
                        rng.choice([rng.randrange(0, 40), rng.randrange(1, 300), rng.randrange(1, 900),
                                    128 * rng.randrange(1, 5), 64 * rng.randrange(1, 8) + rng.choice([-1, 1])]))
                    for _ in range(rng.randrange(1, 10))]
            if sum(lens) == 0:
                lens.append(5)
            _check_varlen(H, D, lens, dtype, ac, seed=seed)
