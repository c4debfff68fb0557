"""The attention weights themselves (the reference forward's `return_attention` debug output, sb_fwd.py:141-172 and
sb_varlen_fwd.py:409-446) against the oracle's attention matrix: fp32 arithmetic on the given inputs, so the bound
is the fp32 one (1e-4 absolute; weights lie in [0, 1])."""
import math

import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, max_abs, cu_from_lengths

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("T,D", [(1, 64), (200, 64), (333, 80), (129, 256)])
def test_dense_weights_match_the_oracle_matrix(T, D, dtype, attend_current):
    from flame_amd.stickbreaking_attention.sb_attn import attention_weights
    from flame_amd import sb_attn
    q, k, v = (randn((2, 3, T, D), 700 + i + T, 0.5, dtype) for i in range(3))
    print(f"weights dense T{T} D{D} {dtype} ac={attend_current}", flush=True)
    W = attention_weights(q.cuda(), k.cuda(), attend_current=attend_current)
    A, rem = O._attention_matrix(q, k, 1 / math.sqrt(D), attend_current, torch.float32)
    assert W.dtype == torch.float32 and W.shape == (2, 3, T, T)
    assert max_abs(W.cpu(), A) <= TOL
    assert torch.count_nonzero(W.cpu()[..., O.causal_mask(T, attend_current)]) == 0      # nothing written outside the mask
    assert max_abs(1 - W.sum(-1).cpu(), rem) <= 2e-4                      # what is left over is rem
    # and they are the weights the operator itself uses, to its own tolerance
    o, _ = sb_attn(q.cuda(), k.cuda(), v.cuda(), attend_current=attend_current)
    tol = {torch.bfloat16: 2e-2, torch.float16: 2.5e-3, torch.float32: 1e-4}[dtype]
    assert max_abs(o.float(), W @ v.cuda().float()) <= tol


def test_packed_weights_are_the_documents_blocks_on_the_diagonal():
    from flame_amd.stickbreaking_attention.sb_varlen import attention_weights_varlen
    lens = [70, 0, 1, 200, 129]
    cu = cu_from_lengths(lens)
    H, D, N = 3, 64, sum(lens)
    q, k = (randn((H, N, D), 720 + i, 0.5, torch.bfloat16) for i in range(2))
    W = attention_weights_varlen(q.cuda(), k.cuda(), cu.cuda(), max(lens)).cpu()
    assert W.shape == (H, N, N)
    expect = torch.zeros(H, N, N)
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        if b > a:
            expect[:, a:b, a:b] = O._attention_matrix(q[:, a:b], k[:, a:b], 1 / math.sqrt(D), False, torch.float32)[0]
    assert max_abs(W, expect) <= TOL
    outside = torch.ones(N, N, dtype=torch.bool)
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        outside[a:b, a:b] = O.causal_mask(b - a, False)
    assert torch.count_nonzero(W[:, outside]) == 0


def test_the_forward_functions_return_the_weights_as_a_fourth_result_like_the_reference():
    from flame_amd.stickbreaking_attention.sb_attn import _fwd
    from flame_amd.stickbreaking_attention.sb_varlen import varlen_fwd
    q, k, v = (randn((1, 2, 150, 64), 730 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o, rem, _, W = _fwd(q, k, v, 0.125, return_attention=True)
    assert max_abs(o.float(), W @ v.float()) <= 2e-2 and max_abs(rem.float(), 1 - W.sum(-1)) <= 2e-2
    cu = cu_from_lengths([100, 50]).cuda()
    o2, rem2, _, W2 = varlen_fwd(q[0], k[0], v[0], cu, 100, 0.125, return_attention=True)
    assert W2.shape == (2, 150, 150) and torch.count_nonzero(W2[:, 100:, :100]) == 0
    assert max_abs(o2.float(), W2 @ v[0].float()) <= 2e-2
