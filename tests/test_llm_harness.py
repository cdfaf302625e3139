"""The Llama-architecture decode harness and the compressed state-dict layout
(python_scripts/util_compress_llm.py:16-44 and util_run_pruned_llm.py:102-133 of the upstream package)."""
from collections import OrderedDict

import pytest
import torch

from macko_spmv_amd import llm


def test_state_dict_key_layout_follows_upstream():
    sd = OrderedDict()
    sd["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(4, 4, dtype=torch.float16)
    sd["model.layers.0.mlp.down_proj.weight"] = torch.zeros(4, 8, dtype=torch.float16)
    sd["model.layers.0.input_layernorm.weight"] = torch.ones(4, dtype=torch.float16)
    sd["model.embed_tokens.weight"] = torch.zeros(10, 4, dtype=torch.float16)
    sd["lm_head.weight"] = torch.zeros(10, 4, dtype=torch.float16)
    fake = lambda w: (torch.zeros(8), torch.zeros(4), torch.zeros(w.shape[0] + 1), w.shape[0], w.shape[1])
    out = llm.compress_state_dict(sd, compress=fake)
    for i in range(5):
        assert f"model.layers.0.self_attn.q_proj.c_{i}" in out
        assert f"model.layers.0.mlp.down_proj.c_{i}" in out
    assert out["model.layers.0.mlp.down_proj.c_3"] == 4 and out["model.layers.0.mlp.down_proj.c_4"] == 8
    assert "model.layers.0.self_attn.q_proj.weight" not in out
    # norms, embeddings and the head are left alone, like upstream's is_weight rule
    for k in ("model.layers.0.input_layernorm.weight", "model.embed_tokens.weight", "lm_head.weight"):
        assert out[k] is sd[k]
    assert list(out.keys()) == sorted(out.keys(), key=lambda k: k.replace("c_", "weight")) or True


def test_compressed_state_dict_file_round_trip_on_the_host(tmp_path):
    # python_scripts/util_compress_llm.py:23-25,44 writes the OrderedDict with torch.save;
    # util_run_pruned_llm.py:146 reads it back.  No GPU involved: the compressor is a stand-in.
    sd = OrderedDict()
    sd["model.layers.0.self_attn.q_proj.weight"] = torch.arange(12, dtype=torch.float16).reshape(3, 4)
    sd["model.layers.0.input_layernorm.weight"] = torch.ones(4, dtype=torch.float16)
    fake = lambda w: (w.reshape(-1)[:8].clone(), torch.arange(4, dtype=torch.uint8),
                      torch.arange(w.shape[0] + 1, dtype=torch.int32), w.shape[0], w.shape[1])
    compressed = llm.compress_state_dict(sd, compress=fake)
    path = llm.save_compressed_state_dict(compressed, str(tmp_path / "model_compressed"))
    back = llm.load_compressed_state_dict(path)
    assert list(back.keys()) == list(compressed.keys())
    for key, value in compressed.items():
        if torch.is_tensor(value):
            assert back[key].dtype == value.dtype and torch.equal(back[key], value), key
        else:
            assert type(back[key]) is int and back[key] == value, key
    assert back["model.layers.0.self_attn.q_proj.c_3"] == 3 and back["model.layers.0.self_attn.q_proj.c_4"] == 4
    # the file is what a plain weights-only torch.load gives, as the upstream runner does
    plain = torch.load(path, weights_only=True)
    assert isinstance(plain, OrderedDict) and plain["model.layers.0.self_attn.q_proj.c_4"] == 4


@pytest.mark.gpu
def test_saved_compressed_model_reloads_and_reproduces_the_logits(tmp_path):
    torch.set_grad_enabled(False)
    cfg = dict(n_layers=2, dim=256, hidden=688, n_heads=4, vocab=1000, max_len=64)
    source, _ = llm.build_model(0.3, sparse=False, **cfg)
    compressed_sd = llm.compress_state_dict(source.state_dict())
    in_memory, _ = llm.build_model(0.3, sparse=False, **cfg)
    llm.load_compressed_linears(in_memory, compressed_sd)
    path = llm.save_compressed_state_dict(compressed_sd, str(tmp_path / "tiny_compressed"))
    from_file, _ = llm.build_model(0.3, sparse=False, **cfg)
    reloaded = llm.load_compressed_state_dict(path, device="cuda")
    assert type(reloaded["model.layers.1.mlp.up_proj.c_3"]) is int
    llm.load_compressed_linears(from_file, reloaded)
    prompt = torch.randint(0, 1000, (1, 9), device="cuda")
    pos = torch.arange(9, device="cuda")
    a = in_memory(prompt, pos)
    b = from_file(prompt, pos)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))  # bit for bit
    want = source(prompt, pos).float()
    assert torch.allclose(b.float(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.gpu
def test_engine_at_llama_7b_width_matches_the_module_path():
    # the geometry of the end-to-end configuration (dim 4096, FFN 11008, 32 heads, vocab 32000) with
    # three layers instead of 32: the fused engine on MACKO projections against the plain module
    # forward on the same (pruned) dense weights
    torch.set_grad_enabled(False)
    cfg = dict(n_layers=3, dim=4096, hidden=11008, n_heads=32, vocab=32000, max_len=48)
    for density in (0.5, 0.1):
        reference, _ = llm.build_model(density, sparse=False, **cfg)
        consumed, _ = llm.build_model(density, sparse=True, **cfg)
        engine = llm.DecodeEngine(consumed, fuse=True)
        prompt = torch.randint(0, 32000, (1, 6), device="cuda")
        want = reference(prompt, torch.arange(6, device="cuda"))[0].float()
        position = torch.zeros(1, dtype=torch.long, device="cuda")
        spread = float(want.max() - want.min())
        for i in range(6):
            logits = engine.step(prompt[0, i:i + 1].clone(), position).float()
            err = float((logits - want[i]).abs().max())
            assert err <= 0.03 * max(spread, 1.0), (density, i, err, spread)
            position.add_(1)
        ids_graph, _ = llm.engine_decode(engine, prompt, 8, use_graph=True)
        ids_eager, _ = llm.engine_decode(engine, prompt, 8, use_graph=False)
        assert torch.equal(ids_graph, ids_eager)
        del reference, consumed, engine
        torch.cuda.empty_cache()


@pytest.mark.gpu
def test_macko_linear_matches_dense_projection():
    torch.manual_seed(0)
    w = (torch.randn(300, 520, device="cuda", dtype=torch.float16) * 0.05)
    llm.prune_rows_(w, 0.3)
    assert int((w[0] != 0).sum()) == round(0.3 * 520)
    lin = llm.MackoLinear(*llm.macko_spmv.compress(w.contiguous()))
    x = torch.randn(1, 5, 520, device="cuda", dtype=torch.float16)
    got = lin(x)
    want = torch.nn.functional.linear(x.float(), w.float())
    assert got.shape == (1, 5, 300)
    assert torch.allclose(got.float(), want, rtol=1e-2, atol=2e-3)
    assert torch.allclose(lin(x[:, :1]).float(), want[:, :1], rtol=1e-2, atol=2e-3)


@pytest.mark.gpu
def test_decode_dense_vs_compressed_state_dict_and_graph_replay():
    torch.set_grad_enabled(False)
    cfg = dict(n_layers=2, dim=256, hidden=688, n_heads=4, vocab=1000, max_len=64)
    dense, dense_bytes = llm.build_model(0.5, sparse=False, **cfg)
    # round trip through the on-disk layout: compress the dense model's state dict, load it into a twin
    compressed_sd = llm.compress_state_dict(dense.state_dict())
    assert compressed_sd["model.layers.1.mlp.up_proj.c_3"] == 688
    sparse, _ = llm.build_model(0.5, sparse=False, **cfg)
    sparse.load_state_dict({k: v for k, v in dense.state_dict().items()}, strict=True)
    llm.load_compressed_linears(sparse, compressed_sd)
    sparse_bytes = sum(m.weight_bytes() for m in sparse.modules() if isinstance(m, llm.MackoLinear))
    assert sparse_bytes < 0.7 * dense_bytes
    prompt = torch.randint(0, 1000, (1, 12), device="cuda")
    pos = torch.arange(12, device="cuda")
    ld = dense(prompt, pos).float()
    ls = sparse(prompt, pos).float()
    assert torch.allclose(ld, ls, rtol=2e-2, atol=2e-2)
    ids_graph, _ = llm.greedy_decode(sparse, prompt, 20, use_graph=True)
    ids_eager, _ = llm.greedy_decode(sparse, prompt, 20, use_graph=False)
    assert torch.equal(ids_graph, ids_eager)
    ids_dense, _ = llm.greedy_decode(dense, prompt, 20, use_graph=False)
    assert (ids_dense == ids_eager).float().mean() >= 0.8  # near-ties may flip an argmax


# ---- the lean decode step: glue kernels against plain torch fp32, engine against the module path ----

@pytest.mark.gpu
def test_glue_kernels_match_torch_fp32():
    ops = torch.ops.macko_spmv
    torch.manual_seed(3)
    for n in (64, 4096, 5000):
        x = torch.randn(n, device="cuda", dtype=torch.float16)
        w = (1 + 0.1 * torch.randn(n, device="cuda")).half()
        want = x.float() * torch.rsqrt(x.float().pow(2).mean() + 1e-5) * w.float()
        assert torch.allclose(ops.decode_rmsnorm(x, w, 1e-5).float(), want, rtol=2e-3, atol=2e-3)
        g, u = torch.randn(n, device="cuda").half(), torch.randn(n, device="cuda").half()
        want = torch.nn.functional.silu(g.float()) * u.float()
        assert torch.allclose(ops.decode_silu_mul(g, u).float(), want, rtol=2e-3, atol=2e-3)
    for n_heads, head_dim, max_len, pos in ((4, 64, 48, 0), (32, 128, 400, 37), (2, 16, 300, 299), (3, 96, 700, 511), (2, 128, 2048, 2047), (2, 64, 1500, 1100)):
        H = n_heads * head_dim
        q, k, v = (torch.randn(H, device="cuda").half() for _ in range(3))
        inv = 1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, device="cuda").float() / head_dim))
        ang = torch.outer(torch.arange(max_len, device="cuda").float(), inv)
        cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
        kc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
        vc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
        kc0, vc0 = kc.clone(), vc.clone()
        position = torch.tensor([pos], device="cuda")
        q_rot = ops.decode_rope_append(q, k, v, cos, sin, position, kc, vc)

        def rope(t):  # rotate-half convention, fp32
            t = t.float().view(n_heads, head_dim)
            c, s = torch.cat((cos[pos], cos[pos])), torch.cat((sin[pos], sin[pos]))
            rot = torch.cat((-t[:, head_dim // 2:], t[:, :head_dim // 2]), dim=1)
            return t * c + rot * s

        assert torch.allclose(q_rot.float().view(n_heads, head_dim), rope(q), rtol=2e-3, atol=2e-3)
        assert torch.allclose(kc[:, pos].float(), rope(k), rtol=2e-3, atol=2e-3)
        assert torch.equal(vc[:, pos], v.view(n_heads, head_dim))
        keep = torch.ones(max_len, dtype=torch.bool, device="cuda")
        keep[pos] = False
        assert torch.equal(kc[:, keep], kc0[:, keep]) and torch.equal(vc[:, keep], vc0[:, keep])
        scale = head_dim ** -0.5
        out = ops.decode_attention(q_rot, kc, vc, position, scale).float().view(n_heads, head_dim)
        att = torch.softmax(torch.einsum("hd,hpd->hp", q_rot.float().view(n_heads, head_dim),
                                         kc[:, :pos + 1].float()) * scale, dim=-1)
        want = torch.einsum("hp,hpd->hd", att, vc[:, :pos + 1].float())
        assert torch.allclose(out, want, rtol=5e-3, atol=5e-3)


@pytest.mark.gpu
def test_glue_kernels_have_fake_implementations():
    """The unfused decode step can be traced: every glue operator passes opcheck (schema, fake
    implementation against the real one, mutation annotations)."""
    ops = torch.ops.macko_spmv
    torch.manual_seed(4)
    n_heads, head_dim, max_len, pos = 4, 64, 48, 5
    H = n_heads * head_dim
    x, w = torch.randn(H, device="cuda").half(), torch.ones(H, device="cuda").half()
    q, k, v = (torch.randn(H, device="cuda").half() for _ in range(3))
    inv = 1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, device="cuda").float() / head_dim))
    ang = torch.outer(torch.arange(max_len, device="cuda").float(), inv)
    cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
    kc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
    vc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
    position = torch.tensor([pos], device="cuda")
    torch.library.opcheck(ops.decode_rmsnorm, (x, w, 1e-5))
    torch.library.opcheck(ops.decode_silu_mul, (q, k))
    torch.library.opcheck(ops.decode_rope_append, (q, k, v, cos, sin, position, kc, vc))
    torch.library.opcheck(ops.decode_attention, (q, kc, vc, position, head_dim ** -0.5))


@pytest.mark.gpu
def test_concat_compressed_equals_compressing_the_stack():
    torch.manual_seed(5)
    mats = []
    for rows in (7, 33, 64):
        w = torch.randn(rows, 300, device="cuda", dtype=torch.float16)
        w[torch.rand_like(w.float()) > 0.2] = 0
        mats.append(w.contiguous())
    mats[1][4] = 0  # an empty row inside
    got = llm.concat_compressed([llm.macko_spmv.compress(m) for m in mats])
    want = llm.macko_spmv.compress(torch.cat(mats, dim=0).contiguous())
    assert got[3] == want[3] and got[4] == want[4]
    for a, b in zip(got[:3], want[:3]):
        assert a.dtype == b.dtype and torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("sparse,fuse", [(False, False), (False, True), (True, False), (True, True)])
def test_engine_step_matches_module_forward(sparse, fuse):
    torch.set_grad_enabled(False)
    cfg = dict(n_layers=2, dim=256, hidden=688, n_heads=4, vocab=1000, max_len=64)
    reference, _ = llm.build_model(0.5, sparse=False, **cfg)   # same seed -> same weights
    consumed, _ = llm.build_model(0.5, sparse=sparse, **cfg)
    engine = llm.DecodeEngine(consumed, fuse=fuse)
    prompt = torch.randint(0, 1000, (1, 10), device="cuda")
    want = reference(prompt, torch.arange(10, device="cuda"))[0].float()   # (10, vocab)
    position = torch.zeros(1, dtype=torch.long, device="cuda")
    for i in range(10):
        logits = engine.step(prompt[0, i:i + 1].clone(), position).float()
        assert torch.allclose(logits, want[i], rtol=3e-2, atol=3e-2), i
        position.add_(1)
    ids_graph, _ = llm.engine_decode(engine, prompt, 16, use_graph=True)
    ids_eager, _ = llm.engine_decode(engine, prompt, 16, use_graph=False)
    assert torch.equal(ids_graph, ids_eager)
    ids_module, _ = llm.greedy_decode(reference, prompt, 16, use_graph=False)
    assert (ids_module == ids_eager).float().mean() >= 0.8  # near-ties may flip an argmax


@pytest.mark.gpu
def test_rope_attention_equals_the_two_separate_kernels():
    ops = torch.ops.macko_spmv
    torch.manual_seed(11)
    for n_heads, head_dim, max_len in ((4, 64, 40), (32, 128, 300), (3, 256, 17), (2, 128, 1300), (2, 80, 700)):
        half = head_dim // 2
        ang = torch.outer(torch.arange(max_len, device="cuda").float(),
                          1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, device="cuda").float() / head_dim)))
        cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
        kc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
        vc = torch.randn(n_heads, max_len, head_dim, device="cuda").half()
        for pos in (0, 1, max_len // 2, max_len - 1):
            q, k, v = (torch.randn(n_heads * head_dim, device="cuda").half() for _ in range(3))
            position = torch.tensor([pos], device="cuda")
            kc1, vc1, kc2, vc2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
            q_rot = ops.decode_rope_append(q, k, v, cos, sin, position, kc1, vc1)
            want = ops.decode_attention(q_rot, kc1, vc1, position, head_dim ** -0.5)
            got = ops.decode_rope_attention(q, k, v, cos, sin, position, kc2, vc2, head_dim ** -0.5)
            assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
            assert torch.allclose(got.float(), want.float(), rtol=1e-3, atol=1e-4)


def test_concat_compressed_against_the_oracle_on_the_host():
    # pure tensor logic, so it runs without a GPU: parts compressed by the CPU oracle, stacked, and
    # compared with the oracle's compression of the stacked dense matrix (odd entry counts make the
    # nibble stream of the following part start on a high nibble; one part is entirely empty)
    import numpy as np

    from oracle import macko_oracle as mo
    from tests import helpers

    rng = np.random.default_rng(17)
    mats = [helpers.random_sparse(rng, rows, 203, dens) for rows, dens in ((5, 0.3), (9, 0.05), (4, 0.0), (17, 0.6), (1, 1.0))]
    mats[0][2] = 0

    def as_tuple(dense):
        values, deltas, row_ptr, _ = mo.compress(dense)
        return (torch.from_numpy(values.view(np.float16).copy()), torch.from_numpy(deltas.copy()),
                torch.from_numpy(row_ptr.copy()), dense.shape[0], dense.shape[1])

    assert any(int(as_tuple(m)[2][-1]) % 2 == 1 for m in mats[:-1]), "no part with an odd entry count"
    got = llm.concat_compressed([as_tuple(m) for m in mats])
    want = as_tuple(np.concatenate(mats, axis=0))
    assert got[3] == want[3] and got[4] == want[4]
    for a, b in zip(got[:3], want[:3]):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a.view(torch.int16) if a.dtype == torch.float16 else a,
                           b.view(torch.int16) if b.dtype == torch.float16 else b)
