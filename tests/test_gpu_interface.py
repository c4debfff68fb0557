"""GPU tests of the host interface around the kernels: the cu_seqlens producer feeding the
packed operator, torch.compile on the layer (dense and packed routes), argument handling."""
import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, rel_l2, max_abs, cu_from_lengths

pytestmark = pytest.mark.gpu


def test_token_row_to_cu_seqlens_to_packed_operator_against_oracle():
    # the collator's convention (flame/data.py:389-496): BOS starts, EOS ends, context_len
    # re-chunking; what it produces goes straight into sb_attn_varlen
    from flame_amd import sb_attn_varlen
    from flame_amd.packing import cu_seqlens_from_tokens
    g = torch.Generator().manual_seed(5)
    T, H, D, BOS, EOS = 1500, 4, 64, 1, 2
    ids = torch.randint(3, 100, (1, T), generator=g)
    starts = [0, 40, 42, 300, 777, 1400]
    ids[0, starts] = BOS
    ids[0, [s - 1 for s in starts[1:]] + [T - 1]] = EOS
    cases = [
        cu_seqlens_from_tokens(ids, bos_token_id=BOS),
        cu_seqlens_from_tokens(ids, eos_token_id=EOS),
        cu_seqlens_from_tokens(ids, bos_token_id=BOS, context_len=256),
    ]
    assert cases[0].tolist() == starts + [T] and cases[1].tolist() == starts + [T]
    assert cases[2].dtype == torch.int32 and int((cases[2][1:] - cases[2][:-1]).max()) <= 256
    q, k, v, do = (randn((H, T, D), 400 + i, 0.5 if i < 3 else 1.0, torch.bfloat16) for i in range(4))
    for cu in cases:
        lens = (cu[1:] - cu[:-1]).tolist()
        print(f"packing -> operator: {len(lens)} documents, longest {max(lens)}", flush=True)
        qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn_varlen(qg, kg, vg, cu.cuda(), max(lens))
        torch.autograd.backward([o], [do.cuda()])
        o_ref, rem_ref, dq, dk, dv = O.sb_attn_grads_oracle(q, k, v, do, None, cu_seqlens=cu.tolist())
        assert max_abs(o.float().cpu(), o_ref) <= 2e-2 and max_abs(rem.float().cpu(), rem_ref) <= 2e-2
        for got, ref in ((qg.grad, dq), (kg.grad, dk), (vg.grad, dv)):
            assert rel_l2(got.float().cpu(), ref) <= 5e-2


def test_cpu_cu_seqlens_and_reference_underscore_convention():
    # cu_seqlens may live on the host (no device-to-host sync then); the underscore entry point
    # takes the document ends only, as the reference's does (sb_varlen/__init__.py:81)
    from flame_amd.stickbreaking_attention.sb_varlen import sb_attn_varlen, sb_attn_varlen_
    lens = [70, 1, 200, 129]
    cu = cu_from_lengths(lens)
    q, k, v = (randn((3, sum(lens), 64), 410 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o_dev, r_dev = sb_attn_varlen(q, k, v, cu.cuda(), max(lens))
    o_cpu, r_cpu = sb_attn_varlen(q, k, v, cu, max(lens))
    assert torch.equal(o_dev, o_cpu) and torch.equal(r_dev, r_cpu)
    o_ends, r_ends = sb_attn_varlen_(q, k, v, 0.125, cu[1:].cuda(), max(lens), False)
    assert torch.equal(o_dev, o_ends) and torch.equal(r_dev, r_ends)
    o_nz, _ = sb_attn_varlen(q, k, v, cu[1:].cuda(), max(lens), zero_start=False)
    assert torch.equal(o_dev, o_nz)


def test_argument_errors_are_python_errors():
    from flame_amd import sb_attn, sb_attn_varlen
    q = randn((2, 300, 64), 420, 0.5, torch.bfloat16).cuda()
    cu = torch.tensor([0, 100, 300], dtype=torch.int32)
    with pytest.raises(TypeError, match="share a dtype"):
        sb_attn_varlen(q, q.float(), q, cu, 200)
    with pytest.raises(TypeError, match="float16"):
        sb_attn_varlen(q.double(), q.double(), q.double(), cu, 200)
    with pytest.raises(ValueError, match="head_dim"):
        sb_attn(torch.zeros(1, 1, 8, 264, device="cuda"), torch.zeros(1, 1, 8, 264, device="cuda"),
                torch.zeros(1, 1, 8, 264, device="cuda"))
    with pytest.raises(ValueError, match="longest document"):
        sb_attn_varlen(q, q, q, cu, 150)
    with pytest.raises(ValueError, match="ends at"):
        sb_attn_varlen(q, q, q, torch.tensor([0, 100, 299], dtype=torch.int32), 200)


def test_float16_results_and_gradients_come_back_as_float16():
    # float16 inputs run on the float16 matrix-core kernels; against the oracle at bf16's bounds divided by 8
    from flame_amd import sb_attn, sb_attn_varlen
    from oracle import sb_oracle as O
    from helpers import within, max_abs, rel_l2
    B, H, T, D = 1, 2, 300, 64
    q, k, v, do = (randn((B, H, T, D), 425 + i, 0.5 if i < 3 else 1.0, torch.float16) for i in range(4))
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    assert o.dtype == rem.dtype == torch.float16
    o.backward(do.cuda())
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(q, k, v, do, None)
    within("float16 dense T=300", "o", max_abs(o.float().cpu(), o_ref), 2.5e-3)
    within("float16 dense T=300", "rem", max_abs(rem.float().cpu(), rem_ref), 2.5e-3)
    for name, got, ref in (("dq", qg.grad, dq_ref), ("dk", kg.grad, dk_ref), ("dv", vg.grad, dv_ref)):
        assert got.dtype == torch.float16
        within("float16 dense T=300", name, rel_l2(got.float().cpu(), ref), 6.25e-3)
    cu = torch.tensor([0, 100, 300], dtype=torch.int32)
    ov, rv = sb_attn_varlen(q[0].cuda(), k[0].cuda(), v[0].cuda(), cu, 200)
    assert ov.dtype == torch.float16
    o_doc, _ = sb_attn(q[:, :, 100:].cuda(), k[:, :, 100:].cuda(), v[:, :, 100:].cuda())
    assert torch.equal(ov[:, 100:], o_doc[0])


def test_no_grad_forward_keeps_no_carry_table():
    # an evaluation pass under torch.no_grad() with trainable inputs must not allocate the table
    from flame_amd import sb_attn
    q, k, v = (randn((1, 2, 2048, 64), 430 + i, 0.5, torch.bfloat16).cuda().requires_grad_(True) for i in range(3))
    o_train, _ = sb_attn(q, k, v)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    with torch.no_grad():
        o_eval, _ = sb_attn(q, k, v)
    torch.cuda.synchronize()
    table = 2 * 16 * 17 * 128 * 4                     # what the training forward keeps for this shape
    assert torch.cuda.max_memory_allocated() - base < o_eval.numel() * 2 + 2048 * 2 * 2 + table // 2
    assert torch.equal(o_train, o_eval)


def test_layer_backward_of_the_stacked_projection_needs_no_concatenation(monkeypatch):
    # q, k, v are column slices of the stacked projection's output; the operator lays dq, dk, dv out the same
    # way in one allocation and the layer's split hands that allocation to the projection's backward.  Both
    # routes (dense, packed), against the layer with three separate projections.
    from flame_amd import sba_layer
    from flame_amd.sba_layer import SBA
    handed = []
    found = sba_layer._adjacent_columns
    monkeypatch.setattr(sba_layer, "_adjacent_columns", lambda gs, shape: handed.append(found(gs, shape)) or handed[-1])
    torch.manual_seed(5)
    layer = SBA(hidden_size=256, num_heads=4).cuda().to(torch.bfloat16)
    x = (torch.randn(2, 200, 256, device="cuda") * 0.5).to(torch.bfloat16)
    cu = cu_from_lengths([130, 7, 200, 63]).cuda()
    for kwargs, xin in (({}, x), ({"cu_seqlens": cu}, x.reshape(1, 400, 256))):
        grads = []
        for fused in (True, False):
            layer.fuse_qkv = fused
            layer.zero_grad(set_to_none=True)
            xi = xin.clone().requires_grad_(True)
            o, _, _ = layer(xi, **kwargs)
            o.float().square().sum().backward()
            grads.append([xi.grad.float()] + [p.grad.float() for p in layer.parameters()])
        for a, b in zip(*grads):
            assert rel_l2(a, b) <= 2e-2
    assert len(handed) == 2 and all(h is not None for h in handed)


def test_torch_compile_fullgraph_on_the_layer_dense_and_packed():
    # flame compiles every block (flame/models/parallelize_fla.py:369-403); the layer has to
    # trace as one graph on both routes, and match eager and the oracle
    from flame_amd.sba_layer import SBA
    torch.manual_seed(0)
    layer = SBA(hidden_size=256, num_heads=4).cuda().to(torch.bfloat16)
    x = randn((1, 384, 256), 440, 1.0, torch.bfloat16).cuda()
    w = randn((1, 384, 256), 441, 1.0, torch.bfloat16).cuda()
    cu = torch.tensor([0, 100, 101, 300, 384], dtype=torch.int32, device="cuda")

    def run(fn, **kw):
        layer.zero_grad()
        xx = x.clone().requires_grad_(True)
        o = fn(xx, **kw)[0]
        torch.autograd.backward([o], [w])
        return o, xx.grad, layer.q_proj.weight.grad.clone(), layer.v_proj.weight.grad.clone()

    compiled = torch.compile(layer, fullgraph=True)
    for kw in ({}, {"cu_seqlens": cu, "max_seqlen": 199}):
        print(f"compile layer, packed={bool(kw)}", flush=True)
        eager = run(layer, **kw)
        comp = run(compiled, **kw)
        for a, b in zip(eager, comp):
            assert rel_l2(b.float(), a.float()) <= 1e-2
        # the same layer with the CPU oracle as its attention (fp32)
        ref = SBA(hidden_size=256, num_heads=4)
        ref.load_state_dict({k_: v_.float().cpu() for k_, v_ in layer.state_dict().items()})
        ref.attn_fn = lambda q, k, v, t: O.sb_attn_oracle(q, k, v)
        ref.attn_varlen_fn = lambda q, k, v, c, ml: O.sb_attn_varlen_oracle(q, k, v, c)
        kw_ref = {k_: (v_.cpu() if torch.is_tensor(v_) else v_) for k_, v_ in kw.items()}
        o_ref = ref(x.float().cpu(), **kw_ref)[0]
        assert max_abs(comp[0].float().cpu(), o_ref) <= 3e-2


def test_hf_auto_model_from_config_trains_one_step_on_the_gpu():
    # the route flame's trainer takes for a custom model: AutoModelForCausalLM.from_config on the
    # registered 'sba' config (flame/train.py:66-67, custom_models/sba/__init__.py:7-9)
    from transformers import AutoModelForCausalLM
    import flame_amd.hf as hf
    torch.manual_seed(0)
    cfg = hf.SBAConfig(hidden_size=256, num_hidden_layers=2, num_heads=4, vocab_size=512)
    model = AutoModelForCausalLM.from_config(cfg).cuda()
    assert isinstance(model, hf.SBAForCausalLM)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-3)
    ids = torch.randint(0, 512, (1, 384), device="cuda")
    cu = torch.tensor([0, 100, 101, 300, 384], dtype=torch.int32, device="cuda")
    losses = []
    for _ in range(3):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = model(input_ids=ids, labels=ids, cu_seqlens=cu, max_seqlen=199)
        opt.zero_grad()
        out.loss.backward()
        assert all(torch.isfinite(p.grad).all() for p in model.parameters())
        opt.step()
        losses.append(float(out.loss))
    print("hf losses", losses, flush=True)
    assert losses[-1] < losses[0]
    # and the dense route
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.isfinite(model(input_ids=ids.view(2, 192), labels=ids.view(2, 192)).loss)


def test_hf_auto_model_loss_matches_oracle_attention_packed_and_dense():
    # the HF route held to the oracle like the plain model is: AutoModelForCausalLM.from_config on the GPU
    # (HIP operator, bf16 autocast) against the same weights with the CPU oracle as attention (fp32)
    from transformers import AutoModelForCausalLM
    import flame_amd.hf as hf
    torch.manual_seed(0)
    cfg = hf.SBAConfig(hidden_size=256, num_hidden_layers=2, num_heads=4, vocab_size=512)
    ref = AutoModelForCausalLM.from_config(cfg)
    for layer in ref.model.layers:
        layer.attn.attn_fn = lambda q, k, v, t: O.sb_attn_oracle(q, k, v)
        layer.attn.attn_varlen_fn = lambda q, k, v, cu, ml: O.sb_attn_varlen_oracle(q, k, v, cu)
    gpu = AutoModelForCausalLM.from_config(cfg)
    gpu.load_state_dict(ref.state_dict())
    gpu.cuda()
    ids = torch.randint(0, 512, (1, 384))
    cu = torch.tensor([0, 100, 101, 300, 384], dtype=torch.int32)
    out_ref = ref(input_ids=ids, labels=ids, cu_seqlens=cu)
    out_ref_dense = ref(input_ids=ids.view(2, 192), labels=ids.view(2, 192))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = gpu(input_ids=ids.cuda(), labels=ids.cuda(), cu_seqlens=cu.cuda(), max_seqlen=199)
        out_dense = gpu(input_ids=ids.view(2, 192).cuda(), labels=ids.view(2, 192).cuda())
    print("hf vs oracle: packed", float(out.loss), float(out_ref.loss), "dense", float(out_dense.loss), float(out_ref_dense.loss), flush=True)
    assert abs(float(out.loss) - float(out_ref.loss)) <= 2e-2
    assert abs(float(out_dense.loss) - float(out_ref_dense.loss)) <= 2e-2
    assert max_abs(out.logits.float().cpu(), out_ref.logits) <= 5e-2
    assert max_abs(out_dense.logits.float().cpu(), out_ref_dense.logits) <= 5e-2
    # the gradients of the attention projections against the oracle's (the operator's backward on this route)
    out.loss.backward()
    out_ref.loss.backward()
    for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
        g = getattr(gpu.model.layers[0].attn, name).weight.grad.float().cpu()
        r = getattr(ref.model.layers[0].attn, name).weight.grad
        assert rel_l2(g, r) <= 5e-2, name
