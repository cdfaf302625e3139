"""Llama-architecture batch-1 decode with MACKO linear layers.

Counterpart of the upstream helper scripts:
  python_scripts/util_compress_llm.py:16-44    -> compress_state_dict()  (keys `<module>.c_0 .. c_4`),
                                                  save_compressed_state_dict() / load_compressed_state_dict()
  python_scripts/util_run_pruned_llm.py:102-133 -> MackoLinear (their CustomLayer), load_compressed_linears (their fix)
  python_scripts/util_run_pruned_llm.py:51-99,136-207 -> Generator-style greedy decode loop and the tok/s, memory report

The upstream scripts wrap a Hugging Face checkpoint and tokenizer fetched by name; neither exists
offline, so the model here is a self-contained decoder with the same architecture and the same
parameter names (`model.layers.{i}.self_attn.q_proj.weight`, ...), randomly initialised, and the
prompt is random token ids.  Decode steps are captured in a HIP graph (the upstream script uses
torch.compile(mode="reduce-overhead") for the same purpose).

Run:  python -m macko_spmv_amd.llm --density 0.5            (prints one JSON line)
"""
import argparse
import json
import math
import sys
import time
from collections import OrderedDict

import torch
from torch import nn

import macko_spmv_amd as macko_spmv

PROJECTIONS = (("self_attn", "q_proj"), ("self_attn", "k_proj"), ("self_attn", "v_proj"), ("self_attn", "o_proj"),
               ("mlp", "gate_proj"), ("mlp", "up_proj"), ("mlp", "down_proj"))


def is_compressible(key):
    """Same rule as upstream compress_k: attention and MLP weight matrices only."""
    return ("weight" in key) and ("self_attn" in key or "mlp" in key)


def compress_state_dict(state_dict, compress=None):
    """state_dict -> OrderedDict where every compressible `<m>.weight` became `<m>.c_0 .. <m>.c_4`
    (values, deltas, row_indices, rows, cols); other entries pass through.  Keys are visited in
    sorted order like upstream."""
    compress = compress or macko_spmv.compress
    out = OrderedDict()
    for key in sorted(state_dict.keys()):
        value = state_dict[key]
        if is_compressible(key):
            compressed = compress(value.contiguous())
            for i in range(5):
                out[key.replace("weight", f"c_{i}")] = compressed[i]
        else:
            out[key] = value
    return out


def save_compressed_state_dict(compressed_sd, path):
    """Write a compressed state dict the way the upstream script does: one torch.save of an
    OrderedDict whose `<m>.c_0 .. c_2` are tensors and `<m>.c_3`, `<m>.c_4` Python ints
    (python_scripts/util_compress_llm.py:23-25,44).  Tensors are moved to the CPU first, so the
    file loads on a host without a GPU."""
    out = OrderedDict()
    for key, value in compressed_sd.items():
        if torch.is_tensor(value):
            out[key] = value.detach().cpu().contiguous()
        else:
            out[key] = int(value)
    torch.save(out, path)
    return path


def load_compressed_state_dict(path, device=None):
    """Read a file written by save_compressed_state_dict or by the upstream script
    (python_scripts/util_run_pruned_llm.py:146 does a plain torch.load).  Loaded with
    weights_only=True: nothing in the file is executed.  Tensors go to `device` if given; the
    `c_3` / `c_4` entries come back as Python ints."""
    loaded = torch.load(path, map_location="cpu", weights_only=True)
    out = OrderedDict()
    for key, value in loaded.items():
        if torch.is_tensor(value):
            out[key] = value.to(device) if device is not None else value
        else:
            out[key] = int(value)
    return out


class MackoLinear(nn.Module):
    """y = M x for a compressed M; x of shape (..., cols) -> (..., rows)."""

    def __init__(self, c_0, c_1, c_2, c_3, c_4):
        super().__init__()
        self.register_buffer("c_0", c_0)
        self.register_buffer("c_1", c_1)
        self.register_buffer("c_2", c_2)
        self.c_3 = int(c_3)
        self.c_4 = int(c_4)

    def forward(self, x):
        lead = x.shape[:-1]
        flat = x.reshape(-1, self.c_4)
        compressed = (self.c_0, self.c_1, self.c_2, self.c_3, self.c_4)
        if flat.shape[0] == 1:
            out = macko_spmv.multiply(compressed, flat[0].contiguous()).unsqueeze(0)
        else:  # all rows of x in one call; upstream maps the single-vector operator over them (vmap)
            out = macko_spmv.multiply_batched(compressed, flat.contiguous())
        return out.reshape(*lead, self.c_3)

    def weight_bytes(self):
        return self.c_0.numel() * 2 + self.c_1.numel() + self.c_2.numel() * 4


def load_compressed_linears(model, compressed_sd):
    """Swap the seven projections of every layer for MackoLinear built from `compressed_sd`."""
    for i, layer in enumerate(model.model.layers):
        for parent, name in PROJECTIONS:
            path = f"model.layers.{i}.{parent}.{name}"
            setattr(getattr(layer, parent), name,
                    MackoLinear(*[compressed_sd[f"{path}.c_{k}"] for k in range(5)]))
    return model


# ---- a minimal Llama-architecture decoder (batch 1) ------------------------------------------------

class RMSNorm(nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        v = x.float()
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
        return (v * self.weight.float()).to(x.dtype)


class Attention(nn.Module):
    def __init__(self, dim, n_heads, max_len):
        super().__init__()
        self.n_heads, self.head_dim, self.max_len = n_heads, dim // n_heads, max_len
        self.q_proj = nn.Linear(dim, dim, bias=False)
        self.k_proj = nn.Linear(dim, dim, bias=False)
        self.v_proj = nn.Linear(dim, dim, bias=False)
        self.o_proj = nn.Linear(dim, dim, bias=False)
        self.register_buffer("k_cache", torch.zeros(1, n_heads, max_len, self.head_dim), persistent=False)
        self.register_buffer("v_cache", torch.zeros(1, n_heads, max_len, self.head_dim), persistent=False)

    def forward(self, x, cos, sin, positions, mask):
        t = x.shape[1]
        q = self.q_proj(x).view(1, t, self.n_heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(x).view(1, t, self.n_heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(x).view(1, t, self.n_heads, self.head_dim).transpose(1, 2)
        q, k = _rope(q, cos, sin), _rope(k, cos, sin)
        self.k_cache.index_copy_(2, positions, k)
        self.v_cache.index_copy_(2, positions, v)
        att = torch.matmul(q, self.k_cache.transpose(2, 3)) / math.sqrt(self.head_dim)
        att = torch.softmax((att + mask).float(), dim=-1).to(x.dtype)
        out = torch.matmul(att, self.v_cache).transpose(1, 2).reshape(1, t, -1)
        return self.o_proj(out)


def _rope(x, cos, sin):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return x * cos + torch.cat((-x2, x1), dim=-1) * sin


class MLP(nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.gate_proj = nn.Linear(dim, hidden, bias=False)
        self.up_proj = nn.Linear(dim, hidden, bias=False)
        self.down_proj = nn.Linear(hidden, dim, bias=False)

    def forward(self, x):
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class Block(nn.Module):
    def __init__(self, dim, hidden, n_heads, max_len):
        super().__init__()
        self.self_attn = Attention(dim, n_heads, max_len)
        self.mlp = MLP(dim, hidden)
        self.input_layernorm = RMSNorm(dim)
        self.post_attention_layernorm = RMSNorm(dim)

    def forward(self, x, cos, sin, positions, mask):
        x = x + self.self_attn(self.input_layernorm(x), cos, sin, positions, mask)
        return x + self.mlp(self.post_attention_layernorm(x))


class _Body(nn.Module):
    def __init__(self, vocab, dim, hidden, n_layers, n_heads, max_len):
        super().__init__()
        self.embed_tokens = nn.Embedding(vocab, dim)
        self.layers = nn.ModuleList([Block(dim, hidden, n_heads, max_len) for _ in range(n_layers)])
        self.norm = RMSNorm(dim)


class LlamaDecoder(nn.Module):
    """Parameter names follow the Hugging Face Llama layout so compressed state dicts are
    interchangeable with the upstream scripts' (`model.layers.{i}.mlp.up_proj.c_0`, ...)."""

    def __init__(self, vocab=32000, dim=4096, hidden=11008, n_layers=32, n_heads=32, max_len=512):
        super().__init__()
        self.max_len, self.head_dim = max_len, dim // n_heads
        self.model = _Body(vocab, dim, hidden, n_layers, n_heads, max_len)
        self.lm_head = nn.Linear(dim, vocab, bias=False)
        inv = 1.0 / (10000.0 ** (torch.arange(0, self.head_dim, 2).float() / self.head_dim))
        ang = torch.outer(torch.arange(max_len).float(), inv)
        ang = torch.cat((ang, ang), dim=-1)
        self.register_buffer("cos", ang.cos(), persistent=False)
        self.register_buffer("sin", ang.sin(), persistent=False)

    def forward(self, tokens, positions):
        """tokens (1, t) int64, positions (t,) int64 -> logits (1, t, vocab)."""
        x = self.model.embed_tokens(tokens)
        cos = self.cos[positions].to(x.dtype)[None, None]
        sin = self.sin[positions].to(x.dtype)[None, None]
        key_pos = torch.arange(self.max_len, device=tokens.device)
        mask = torch.where(key_pos[None, :] <= positions[:, None], 0.0, float("-inf")).to(x.dtype)[None, None]
        for layer in self.model.layers:
            x = layer(x, cos, sin, positions, mask)
        return self.lm_head(self.model.norm(x))


def prune_rows_(weight, density):
    """In place: keep the round(density * cols) largest |w| of every row."""
    keep = int(round(density * weight.shape[1]))
    if keep < weight.shape[1]:
        idx = weight.abs().float().topk(keep, dim=1).indices
        mask = torch.zeros_like(weight, dtype=torch.bool)
        mask.scatter_(1, idx, True)
        weight.mul_(mask)
    return weight


@torch.no_grad()
def greedy_decode(model, prompt, new_tokens, use_graph=True):
    """Prefill `prompt` (1, t), then generate `new_tokens` greedily, one token per step.
    Returns (generated ids (new_tokens,), seconds spent in the decode steps)."""
    device = prompt.device
    t = prompt.shape[1]
    logits = model(prompt, torch.arange(t, device=device))
    token = logits[:, -1].argmax(-1, keepdim=True)           # (1, 1)
    position = torch.tensor([t], device=device)
    out = torch.zeros(new_tokens, dtype=torch.long, device=device)
    out[0] = token[0, 0]

    def step():
        nxt = model(token, position)[:, -1].argmax(-1, keepdim=True)
        token.copy_(nxt)
        position.add_(1)

    graph = None
    if use_graph:
        state = (token.clone(), position.clone())
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()                                            # warm-up outside capture
            side.synchronize()
            token.copy_(state[0])
            position.copy_(state[1])
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                step()
            token.copy_(state[0])
            position.copy_(state[1])
        torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for i in range(1, new_tokens):
        if graph is not None:
            graph.replay()
        else:
            step()
        out[i] = token[0, 0]
    torch.cuda.synchronize()
    return out, time.perf_counter() - start


# ---- a lean single-token decode step ----------------------------------------------------------------

def concat_compressed(parts):
    """Stack compressed matrices with equal column counts row-wise.  The result is bit-identical to
    compressing the row-wise concatenation of the dense matrices (rows are compressed independently;
    only the nibble stream has to be re-packed when a part holds an odd number of entries)."""
    cols = parts[0][4]
    assert all(p[4] == cols for p in parts)
    values, nibbles, row_ptrs, base, rows = [], [], [parts[0][2].new_zeros(1)], 0, 0
    for v, d, rp, r, _ in parts:
        n = int(rp[-1].item())
        values.append(v[:n])
        nibbles.append(torch.stack((d & 15, d >> 4), dim=1).reshape(-1)[:n])
        row_ptrs.append(rp[1:] + base)
        base += n
        rows += r
    pad = (-base) % 8
    values = torch.cat(values + [values[0].new_zeros(pad)])
    nib = torch.cat(nibbles + [nibbles[0].new_zeros(pad)]).view(-1, 2)
    deltas = (nib[:, 0] | (nib[:, 1] << 4)).contiguous()
    return values.contiguous(), deltas, torch.cat(row_ptrs).contiguous(), rows, cols


class DecodeEngine:
    """One token in, logits out, with as few launches as the architecture allows: q|k|v and gate|up
    stacked into one matrix each, residual additions folded into the o_proj / down_proj products
    (y = Mx + y), and the parts between the products (RMSNorm, rotary + KV-cache append, attention,
    SiLU * up) as one hand-written kernel each.  Works on a LlamaDecoder whose projections are either
    nn.Linear (dense) or MackoLinear; the model's projection modules are consumed (set to None) so
    the weights are held once.

    With fuse=True (the default) a step drops to five launches per layer: rotary, cache append and
    attention share one kernel, and, for MACKO projections, the two RMS norms and the SiLU gate are
    applied by the product that consumes them while it stages its input (multiply_rmsnorm,
    multiply_silu_mul_axpby).  Dense projections go through the BLAS matrix-vector product, which
    has no such hook, and keep their separate norm and gate kernels."""

    def __init__(self, model, fuse=True):
        ops = torch.ops.macko_spmv
        self.ops = ops
        self.fuse = fuse
        body = model.model
        first = body.layers[0].self_attn
        self.n_heads, self.head_dim, self.max_len = first.n_heads, first.head_dim, first.max_len
        self.scale = 1.0 / math.sqrt(self.head_dim)
        dev = body.embed_tokens.weight.device
        half = self.head_dim // 2
        inv = 1.0 / (10000.0 ** (torch.arange(0, self.head_dim, 2, device=dev).float() / self.head_dim))
        ang = torch.outer(torch.arange(self.max_len, device=dev).float(), inv)
        assert ang.shape == (self.max_len, half)
        self.cos, self.sin = ang.cos().contiguous(), ang.sin().contiguous()
        self.embed = body.embed_tokens.weight.data
        self.final_norm = body.norm.weight.data.contiguous()
        self.eps = body.norm.eps
        self.lm_head = model.lm_head.weight.data
        self.layers = []
        for layer in body.layers:
            att, mlp = layer.self_attn, layer.mlp
            entry = {
                "norm1": layer.input_layernorm.weight.data.contiguous(),
                "norm2": layer.post_attention_layernorm.weight.data.contiguous(),
                "qkv": self._fuse([att.q_proj, att.k_proj, att.v_proj]),
                "o": self._fuse([att.o_proj]),
                "gate_up": self._fuse([mlp.gate_proj, mlp.up_proj]),
                "down": self._fuse([mlp.down_proj]),
                "k_cache": torch.zeros(self.n_heads, self.max_len, self.head_dim, dtype=torch.float16, device=dev),
                "v_cache": torch.zeros(self.n_heads, self.max_len, self.head_dim, dtype=torch.float16, device=dev),
            }
            att.q_proj = att.k_proj = att.v_proj = att.o_proj = None
            mlp.gate_proj = mlp.up_proj = mlp.down_proj = None
            att.k_cache = att.v_cache = None
            self.layers.append(entry)
        self.dim = self.embed.shape[1]
        self.hidden = self.layers[0]["gate_up"][3] // 2 if isinstance(self.layers[0]["gate_up"], tuple) \
            else self.layers[0]["gate_up"].shape[0] // 2

    @staticmethod
    def _fuse(mods):
        if isinstance(mods[0], MackoLinear):
            parts = [(m.c_0, m.c_1, m.c_2, m.c_3, m.c_4) for m in mods]
            return parts[0] if len(parts) == 1 else concat_compressed(parts)
        ws = [m.weight.data for m in mods]
        return ws[0].contiguous() if len(ws) == 1 else torch.cat(ws, dim=0).contiguous()

    @staticmethod
    def _matvec(W, x):
        if isinstance(W, tuple):
            return macko_spmv.multiply(W, x)
        return torch.mv(W, x)

    @staticmethod
    def _matvec_add(W, x, residual):
        """residual += W x, in place."""
        if isinstance(W, tuple):
            macko_spmv.multiply_axpby(W, x, residual, 1.0, 1.0)
        else:
            residual.addmv_(W, x)

    def weight_bytes(self):
        total = 0
        for entry in self.layers:
            for key in ("qkv", "o", "gate_up", "down"):
                W = entry[key]
                total += (W[0].numel() * 2 + W[1].numel() + W[2].numel() * 4) if isinstance(W, tuple) else W.numel() * 2
        return total

    def step(self, token, position):
        """token (1,) int64, position (1,) int64, both on the GPU -> logits (vocab,) fp16."""
        ops, H, I = self.ops, self.dim, self.hidden
        x = self.embed.index_select(0, token).view(-1)
        for L in self.layers:
            sparse = self.fuse and isinstance(L["qkv"], tuple)
            if sparse:
                qkv = macko_spmv.multiply_rmsnorm(L["qkv"], x, L["norm1"], self.eps)
            else:
                qkv = self._matvec(L["qkv"], ops.decode_rmsnorm(x, L["norm1"], self.eps))
            if self.fuse:
                a = ops.decode_rope_attention(qkv[:H], qkv[H:2 * H], qkv[2 * H:], self.cos, self.sin, position,
                                              L["k_cache"], L["v_cache"], self.scale)
            else:
                q = ops.decode_rope_append(qkv[:H], qkv[H:2 * H], qkv[2 * H:], self.cos, self.sin, position,
                                           L["k_cache"], L["v_cache"])
                a = ops.decode_attention(q, L["k_cache"], L["v_cache"], position, self.scale)
            self._matvec_add(L["o"], a, x)
            if sparse:
                gu = macko_spmv.multiply_rmsnorm(L["gate_up"], x, L["norm2"], self.eps)
                macko_spmv.multiply_silu_mul_axpby(L["down"], gu[:I], gu[I:], x, 1.0, 1.0)
            else:
                gu = self._matvec(L["gate_up"], ops.decode_rmsnorm(x, L["norm2"], self.eps))
                self._matvec_add(L["down"], ops.decode_silu_mul(gu[:I], gu[I:]), x)
        return torch.mv(self.lm_head, ops.decode_rmsnorm(x, self.final_norm, self.eps))


def engine_decode(engine, prompt, new_tokens, use_graph=True):
    """Feed `prompt` (1, t) token by token, then generate `new_tokens` greedily.  Returns
    (generated ids (new_tokens,), seconds spent generating)."""
    device = prompt.device
    t = prompt.shape[1]
    token = prompt[0, :1].clone()
    position = torch.zeros(1, dtype=torch.long, device=device)

    def step():
        nxt = engine.step(token, position).argmax(-1, keepdim=True)
        token.copy_(nxt)
        position.add_(1)

    run = step
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()                                            # warm-up outside capture (position 0)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                step()
        torch.cuda.current_stream().wait_stream(side)
        run = graph.replay
    position.zero_()
    for i in range(t):                                        # prefill: same step, the prediction is discarded
        token.copy_(prompt[0, i:i + 1])
        run()
    out = torch.zeros(new_tokens, dtype=torch.long, device=device)
    out[0] = token[0]
    torch.cuda.synchronize()
    start = time.perf_counter()
    for i in range(1, new_tokens):
        run()
        out[i] = token[0]
    torch.cuda.synchronize()
    return out, time.perf_counter() - start


def build_model(density, n_layers, dim, hidden, n_heads, vocab, max_len, seed=0, sparse=True):
    """Random Llama-architecture fp16 model on the GPU with every projection pruned per row to
    `density`; with sparse=True the projections are replaced by MackoLinear.  Returns (model, bytes
    held by the projection weights)."""
    torch.manual_seed(seed)
    model = LlamaDecoder(vocab, dim, hidden, n_layers, n_heads, max_len).half().cuda()
    proj_bytes = 0
    for i, layer in enumerate(model.model.layers):
        for parent, name in PROJECTIONS:
            lin = getattr(getattr(layer, parent), name)
            w = lin.weight.data
            w.normal_(0.0, 0.02)
            if density < 1.0:
                prune_rows_(w, density)
            if sparse:
                new = MackoLinear(*macko_spmv.compress(w.contiguous()))
                setattr(getattr(layer, parent), name, new)
                proj_bytes += new.weight_bytes()
            else:
                proj_bytes += w.numel() * 2
    torch.cuda.empty_cache()
    return model, proj_bytes


def main(argv=None):
    ap = argparse.ArgumentParser(description="batch-1 greedy decode, dense vs MACKO projections")
    ap.add_argument("--density", type=float, default=0.5)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--dim", type=int, default=4096)
    ap.add_argument("--hidden", type=int, default=11008)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--tokens", type=int, default=256)
    ap.add_argument("--runs", type=int, default=3)
    ap.add_argument("--skip-dense", action="store_true")
    ap.add_argument("--module-path", action="store_true",
                    help="decode through the nn.Module forward (one framework kernel per elementary op) "
                         "instead of the lean DecodeEngine step")
    ap.add_argument("--compressed-file", default=None,
                    help="write the MACKO model's compressed state dict to this file and build the model that "
                         "is timed from what is read back (the upstream pair of scripts: compress to disk, run "
                         "from disk)")
    ap.add_argument("--no-fuse", action="store_true",
                    help="engine path: keep rotary, the RMS norms and the SiLU gate as launches of their own")
    args = ap.parse_args(argv)
    result = measure(density=args.density, layers=args.layers, dim=args.dim, hidden=args.hidden, heads=args.heads,
                     vocab=args.vocab, prompt=args.prompt, tokens=args.tokens, runs=args.runs,
                     skip_dense=args.skip_dense, module_path=args.module_path, compressed_file=args.compressed_file,
                     fuse=not args.no_fuse)
    print(json.dumps(result), flush=True)


def measure(density=0.5, layers=32, dim=4096, hidden=11008, heads=32, vocab=32000, prompt=128, tokens=256, runs=3,
            skip_dense=False, module_path=False, compressed_file=None, fuse=True):
    """Builds the random-init model (dense, then with MACKO projections pruned to `density`), decodes
    `tokens` tokens greedily behind a `prompt`-token prompt and returns tokens/s and memory figures
    (the measurement of python_scripts/util_run_pruned_llm.py:201-207 upstream)."""
    assert torch.cuda.is_available(), "needs a GPU"
    torch.set_grad_enabled(False)
    max_len = prompt + tokens + 8
    torch.cuda.empty_cache()
    held_before = torch.cuda.memory_allocated()  # what the caller keeps on the device is not the model's
    result = {"density": density, "layers": layers, "prompt": prompt, "tokens": tokens,
              "path": "module" if module_path else "engine",
              "fused": not (module_path or not fuse)}
    for label, sparse in (("dense", False), ("macko", True)):
        if label == "dense" and skip_dense:
            continue
        model, proj_bytes = build_model(density, layers, dim, hidden, heads, vocab,
                                        max_len, sparse=sparse and not compressed_file)
        if sparse and compressed_file:
            save_compressed_state_dict(compress_state_dict(model.state_dict()), compressed_file)
            load_compressed_linears(model, load_compressed_state_dict(compressed_file, device="cuda"))
            proj_bytes = sum(m.weight_bytes() for m in model.modules() if isinstance(m, MackoLinear))
            torch.cuda.empty_cache()
        engine = None
        if not module_path:
            engine = DecodeEngine(model, fuse=fuse)
            proj_bytes = engine.weight_bytes()
            torch.cuda.empty_cache()
        resident = torch.cuda.memory_allocated() - held_before
        torch.cuda.reset_peak_memory_stats()  # the peak below covers prefill + decode, not model construction
        g = torch.Generator(device="cuda")
        g.manual_seed(1)
        prompt_ids = torch.randint(0, vocab, (1, prompt), device="cuda", generator=g)
        times = []
        for _ in range(runs):
            if engine is not None:
                ids, seconds = engine_decode(engine, prompt_ids, tokens)
            else:
                ids, seconds = greedy_decode(model, prompt_ids, tokens)
            times.append(seconds)
        best = min(times)
        result[label] = {
            "tokens_per_s": round((tokens - 1) / best, 2),
            "projection_weights_gb": round(proj_bytes / 1e9, 3),
            "model_memory_gb": round(resident / 1e9, 3),
            "peak_memory_gb": round((torch.cuda.max_memory_allocated() - held_before) / 1e9, 3),
            "first_tokens": ids[:8].tolist(),
        }
        print(label, result[label], file=sys.stderr, flush=True)
        del model, engine
        torch.cuda.empty_cache()
    if "dense" in result and "macko" in result:
        result["speedup"] = round(result["macko"]["tokens_per_s"] / result["dense"]["tokens_per_s"], 3)
    return result


if __name__ == "__main__":
    main()
