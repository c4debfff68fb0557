"""Host-side logic around the operator: the SBA layer/model wiring (with the CPU oracle
standing in for the HIP operator) and the cu_seqlens convention."""
import pytest
import torch

from flame_amd.modeling_sba import SBAConfig, SBAForCausalLM
from flame_amd.packing import cu_seqlens_from_tokens, split_by_context_len
from oracle import sb_oracle as O


def _oracle_model(cfg, seed=0):
    torch.manual_seed(seed)
    m = SBAForCausalLM(cfg)
    for layer in m.model.layers:
        layer.attn.attn_fn = lambda q, k, v, t: O.sb_attn_oracle(q, k, v)
        layer.attn.attn_varlen_fn = lambda q, k, v, cu, ml: O.sb_attn_varlen_oracle(q, k, v, cu)
    return m


def test_340m_config_shape():
    cfg = SBAConfig()
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_heads, cfg.vocab_size) == (1024, 24, 16, 32000)
    assert cfg.mlp_width() == 2816
    n = 32000 * 1024 * 2 + 24 * (4 * 1024 * 1024 + 3 * 1024 * 2816 + 2 * 1024) + 1024
    assert abs(n / 1e6 - 373.9) < 0.1          # ~374 M parameters


def test_model_wiring_dense_vs_packed_single_document():
    cfg = SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97)
    m = _oracle_model(cfg)
    ids = torch.randint(0, 97, (1, 40))
    loss_dense, logits_dense = m(ids, labels=ids)
    loss_packed, logits_packed = m(ids, labels=ids, cu_seqlens=torch.tensor([0, 40]))
    assert torch.allclose(logits_dense, logits_packed, atol=1e-5)
    assert torch.allclose(loss_dense, loss_packed, atol=1e-6)
    loss_dense.backward()
    assert all(torch.isfinite(p.grad).all() for p in m.parameters())


def test_packed_documents_do_not_see_each_other():
    cfg = SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97)
    m = _oracle_model(cfg)
    a, b = torch.randint(0, 97, (1, 17)), torch.randint(0, 97, (1, 23))
    _, la = m(a)
    _, lb = m(b)
    _, lab = m(torch.cat([a, b], 1), cu_seqlens=torch.tensor([0, 17, 40]))
    assert torch.allclose(lab[:, :17], la, atol=1e-5) and torch.allclose(lab[:, 17:], lb, atol=1e-5)


def test_stacked_projections_equal_the_separate_ones():
    # q/k/v (and gate/up) run as one product on stacked weights: same logits, same loss, and the same gradient
    # for every one of the separate parameters, with and without biases
    from flame_amd import modeling_sba as M
    for bias in (False, True):
        cfg = SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97, qkv_bias=bias)
        m = _oracle_model(cfg, seed=3)
        if bias:
            for layer in m.model.layers:
                for proj in (layer.attn.q_proj, layer.attn.k_proj, layer.attn.v_proj):
                    torch.nn.init.normal_(proj.bias, std=0.1)
        ids = torch.randint(0, 97, (2, 21))
        results = []
        for fused in (True, False):
            for layer in m.model.layers:
                layer.attn.fuse_qkv = fused
            mlp_forward = M.SBAMLP.forward
            if not fused:
                M.SBAMLP.forward = lambda self, x: self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))
            try:
                m.zero_grad(set_to_none=True)
                loss, logits = m(ids, labels=ids)
                loss.backward()
            finally:
                M.SBAMLP.forward = mlp_forward
            results.append((loss.detach(), logits.detach(), {n: p.grad.clone() for n, p in m.named_parameters()}))
        (l1, g1, p1), (l2, g2, p2) = results
        assert torch.allclose(l1, l2, atol=1e-6) and torch.allclose(g1, g2, atol=1e-5)
        assert p1.keys() == p2.keys()
        for n in p1:
            assert torch.allclose(p1[n], p2[n], atol=1e-5, rtol=1e-4), n


def test_column_split_hands_adjacent_gradients_through_without_a_copy():
    # the q/k/v split of the stacked projection: gradients that already lie side by side in one buffer (how the
    # operator allocates dq, dk, dv for such inputs) go back as that buffer; anything else is concatenated
    from flame_amd import _lib
    from flame_amd.sba_layer import _SplitColumns
    H, D, T = 4, 8, 10
    y = torch.randn(1, T, 3 * H * D, requires_grad=True)
    q, k, v = (x.unflatten(-1, (H, D)).squeeze(0).transpose(0, 1) for x in _SplitColumns.apply(y, H * D, H * D, H * D))
    dq, dk, dv = _lib.empty_grads_like(q.detach(), k.detach(), v.detach())
    assert dq.stride() == q.stride() and dq.untyped_storage().data_ptr() == dv.untyped_storage().data_ptr()
    for t in (dq, dk, dv):
        t.copy_(torch.randn_like(t))
    expect = torch.cat([t.transpose(0, 1).reshape(1, T, H * D) for t in (dq, dk, dv)], -1)
    (g,) = torch.autograd.grad((q, k, v), y, (dq, dk, dv), retain_graph=True)
    assert torch.equal(g, expect) and g.untyped_storage().data_ptr() == dq.untyped_storage().data_ptr()
    # separate allocations, a missing gradient, a different order: the concatenating route, same values
    sep = tuple(t.clone() for t in (dq, dk, dv))
    (g,) = torch.autograd.grad((q, k, v), y, sep, retain_graph=True)
    assert torch.equal(g, expect)
    (g,) = torch.autograd.grad((q, v), y, (dq, dv), retain_graph=True)
    assert torch.equal(g[..., :H * D], expect[..., :H * D]) and not g[..., H * D:2 * H * D].any()
    (g,) = torch.autograd.grad((q, k, v), y, (dk, dq, dv), retain_graph=True)
    assert torch.equal(g[..., :H * D], expect[..., H * D:2 * H * D])
    # tensors that are not slices of one buffer get plain allocations
    a, b, c = _lib.empty_grads_like(torch.zeros(2, 3, 4), torch.zeros(2, 3, 4), torch.zeros(2, 3, 4))
    assert a.is_contiguous() and a.untyped_storage().data_ptr() != b.untyped_storage().data_ptr()


def test_swiglu_function_matches_autograd():
    from flame_amd.modeling_sba import _SwiGLU
    y = torch.randn(3, 5, 12, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_SwiGLU.apply, (y,))
    g, u = y.chunk(2, dim=-1)
    assert torch.equal(_SwiGLU.apply(y), torch.nn.functional.silu(g) * u)


def test_label_shift_ignores_last_position():
    cfg = SBAConfig(hidden_size=32, num_hidden_layers=1, num_heads=2, vocab_size=11)
    m = _oracle_model(cfg)
    ids = torch.randint(0, 11, (2, 9))
    loss, logits = m(ids, labels=ids)
    ref = torch.nn.functional.cross_entropy(logits[:, :-1].reshape(-1, 11), ids[:, 1:].reshape(-1))
    assert torch.allclose(loss, ref, atol=1e-6)


def test_kv_heads_must_equal_heads():
    from flame_amd.sba_layer import SBA
    with pytest.raises(ValueError):
        SBA(hidden_size=64, num_heads=4, num_kv_heads=2)
    # the blocks forward the field (modeling_sba.py:44-53 of the reference does): a config that asks for
    # grouped keys raises instead of silently building full multi-head attention
    with pytest.raises(ValueError):
        SBAForCausalLM(SBAConfig(hidden_size=64, num_hidden_layers=1, num_heads=4, num_kv_heads=2, vocab_size=11))
    import flame_amd.hf as hf
    from transformers import AutoModelForCausalLM
    with pytest.raises(ValueError):
        AutoModelForCausalLM.from_config(hf.SBAConfig(hidden_size=64, num_hidden_layers=1, num_heads=4, num_kv_heads=2,
                                                      vocab_size=11))
    blk = SBAForCausalLM(SBAConfig(hidden_size=64, num_hidden_layers=1, num_heads=4, num_kv_heads=4, window_size=77,
                                   vocab_size=11)).model.layers[0]
    assert blk.attn.num_kv_heads == 4 and blk.attn.window_size == 77      # kept, as the reference layer keeps it


def test_hf_tied_word_embeddings(tmp_path):
    # transformers 5 wants the tie declared as {target: source}; a bare list of names fails in from_config
    import flame_amd.hf as hf
    from transformers import AutoModelForCausalLM
    cfg = hf.SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97, tie_word_embeddings=True)
    lm = AutoModelForCausalLM.from_config(cfg)
    assert lm.lm_head.weight.data_ptr() == lm.model.embeddings.weight.data_ptr()
    n_tied = sum(p.numel() for p in lm.parameters())
    cfg_untied = hf.SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97)
    untied = AutoModelForCausalLM.from_config(cfg_untied)
    assert untied.lm_head.weight.data_ptr() != untied.model.embeddings.weight.data_ptr()
    assert sum(p.numel() for p in untied.parameters()) == n_tied + 97 * 64
    lm.save_pretrained(tmp_path)
    back = AutoModelForCausalLM.from_pretrained(tmp_path)
    assert torch.equal(back.lm_head.weight, lm.lm_head.weight)
    assert back.lm_head.weight.data_ptr() == back.model.embeddings.weight.data_ptr()
    # the plain model ties the same way
    plain = SBAForCausalLM(SBAConfig(hidden_size=64, num_hidden_layers=1, num_heads=2, vocab_size=97, tie_word_embeddings=True))
    assert plain.lm_head.weight is plain.model.embeddings.weight


def test_cu_seqlens_from_bos():
    ids = torch.tensor([[1, 5, 6, 1, 7, 1, 8, 9, 9]])
    assert cu_seqlens_from_tokens(ids, bos_token_id=1).tolist() == [0, 3, 5, 9]
    # a row that does not start with BOS still starts a document at 0
    assert cu_seqlens_from_tokens(ids[:, 1:], bos_token_id=1).tolist() == [0, 2, 4, 8]
    assert cu_seqlens_from_tokens(ids, bos_token_id=1).dtype == torch.int32


def test_cu_seqlens_from_eos():
    ids = torch.tensor([5, 6, 2, 7, 2, 8, 9])
    assert cu_seqlens_from_tokens(ids, eos_token_id=2).tolist() == [0, 3, 5, 7]
    assert cu_seqlens_from_tokens(torch.tensor([5, 6, 2]), eos_token_id=2).tolist() == [0, 3]
    with pytest.raises(ValueError):
        cu_seqlens_from_tokens(ids)


def test_context_len_rechunking():
    cu = torch.tensor([0, 10, 13, 30], dtype=torch.int32)
    assert split_by_context_len(cu, 8).tolist() == [0, 8, 10, 13, 21, 29, 30]
    assert cu_seqlens_from_tokens(torch.tensor([1] + [3] * 19), bos_token_id=1, context_len=8).tolist() == [0, 8, 16, 20]


def test_hf_registration_and_340m_config_values():
    # custom_models/sba/__init__.py:7-9: importing the package registers model_type 'sba'
    import json
    import os
    from transformers import AutoConfig, AutoModel, AutoModelForCausalLM
    import flame_amd.hf as hf
    # the values of the reference's configs/sba_340m.json, read from that file by tests/golden/make_config_fixture.py
    fixture = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sba_340m_config.json")
    sba_340m = json.load(open(fixture))
    cfg = AutoConfig.for_model(**sba_340m)
    for key, value in sba_340m.items():        # every value of the file arrives in the config object
        assert getattr(cfg, key) == value, key
    assert isinstance(cfg, hf.SBAConfig) and cfg.model_type == "sba"
    assert (cfg.hidden_size, cfg.num_heads, cfg.num_hidden_layers, cfg.vocab_size) == (1024, 16, 24, 32000)
    assert cfg.mlp_width() == 2816 and cfg.hidden_ratio == 4 and cfg.norm_eps == 1e-6
    small = hf.SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97)
    lm = AutoModelForCausalLM.from_config(small)
    assert isinstance(lm, hf.SBAForCausalLM) and isinstance(AutoModel.from_config(small), hf.SBAModel)
    # weights are N(0, initializer_range)
    assert abs(float(lm.model.layers[0].attn.q_proj.weight.std()) - 0.006) < 1e-3
    # same wiring as the plain model: the oracle attention in both, equal losses for equal weights
    for layer in lm.model.layers:
        layer.attn.attn_fn = lambda q, k, v, t: O.sb_attn_oracle(q, k, v)
        layer.attn.attn_varlen_fn = lambda q, k, v, cu, ml: O.sb_attn_varlen_oracle(q, k, v, cu)
    plain = _oracle_model(SBAConfig(hidden_size=64, num_hidden_layers=2, num_heads=2, vocab_size=97))
    plain.load_state_dict(lm.state_dict())
    ids = torch.randint(0, 97, (1, 40))
    cu = torch.tensor([0, 17, 40])
    out = lm(input_ids=ids, labels=ids, cu_seqlens=cu)
    loss_plain, logits_plain = plain(ids, labels=ids, cu_seqlens=cu)
    assert torch.allclose(out.logits, logits_plain, atol=1e-5) and torch.allclose(out.loss, loss_plain, atol=1e-6)
