"""Generation harness for the SOCKET decode path: prefill, greedy decode, timing.

Counterpart of GPT-FAST/generate.py (warm-up :28-110, sample :127-132, prefill
:134-140, decode_one_token / sparse_decode_one_token :142-152, decode_n_tokens
:155-189, generate :245-370, _load_model :380-433) with the same function
names and the same accounting (decode-only tokens exclude the token the prefill
produces).  Differences:

  * weights are random (normal, std 0.02) because no checkpoint can be fetched;
    `load_random_model` stands where `_load_model` does;
  * a decode step reads nothing back to the host, so the whole step -- every
    layer, the hash append, score, select, attend and the greedy argmax -- is
    recorded once into a HIP graph and replayed per token (the reference relies
    on torch.compile's "reduce-overhead" mode for its dense path only);
  * timing uses HIP events on the stream the work is issued on.

Run `python -m socket_amd.generate --help` for the command line.
"""
from __future__ import annotations

import argparse
import json
import time
from typing import Callable, List, Optional, Tuple

import torch

from . import hash_cache
from .model import ModelArgs, Transformer
from .socket_kernels import sparse_attention_fwd
from .sparse import select_list


@torch.no_grad()
def warmup_sparse_decode(model: Transformer, device: torch.device, *, T: int = 4096) -> None:
    """Run the step's kernels once on random data of the decode shape so that
    module loading and first-launch costs stay out of the timed region
    (GPT-FAST/generate.py:28-110 does this for its Triton kernels)."""
    attn = model.layers[0].attention
    B, H, Hl, D, L, R, P = 1, attn.n_head, attn.n_local_heads, attn.head_dim, attn.L, attn.R, attn.K
    T = max(int(T), 256)
    Tcap = (T + 7) // 8 * 8
    dtype = model.tok_embeddings.weight.dtype
    q = torch.randn((B, H, D), device=device, dtype=dtype)
    q_probs = torch.rand((B, H, L, R), device=device, dtype=dtype)
    NW = hash_cache.words_per_key(L, P)
    codes = torch.randint(0, 2 ** 31 - 1, (B, Hl, NW, Tcap), device=device, dtype=torch.int32)
    v_norm = torch.rand((B, Hl, Tcap), device=device, dtype=torch.float16)
    k = torch.randn((B, Hl, Tcap, D), device=device, dtype=dtype)
    v = torch.randn((B, Hl, Tcap, D), device=device, dtype=dtype)
    cfg = attn.config
    for _ in range(2):
        hash_cache.sparse_decode_step(q, q_probs, k, v, codes, v_norm, T, P, int(cfg.sink_size),
                                      int(cfg.window_size), int(attn.heavy_const))
    # the library's fixed scratch array is looked up here, outside any capture
    hash_cache.prepare_one_launch_attention(device)
    torch.cuda.synchronize()


def logits_to_probs(logits, temperature: float = 1.0, top_k: Optional[int] = None):
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
        logits = torch.where(logits < v.select(-1, -1).unsqueeze(-1), -float("Inf"), logits)
    return torch.nn.functional.softmax(logits, dim=-1)


def sample(logits, temperature: float = 1.0, top_k: Optional[int] = None):
    """Greedy pick from the last position, as GPT-FAST/generate.py:127-132."""
    probs = logits_to_probs(logits[:, -1], temperature, top_k)
    return torch.argmax(probs, dim=-1, keepdim=True).to(dtype=torch.int), probs


def prefill(model: Transformer, x: torch.Tensor, input_pos: torch.Tensor, decode_type: str,
            **sampling_kwargs) -> torch.Tensor:
    fwd = model.forward if decode_type == "dense" else model.sparse_forward
    logits = fwd(x, input_pos, pos0=0, last_only=True)
    return sample(logits, **sampling_kwargs)[0]


def decode_one_token(model: Transformer, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs):
    assert input_pos.shape[-1] == 1
    return sample(model(x, input_pos), **sampling_kwargs)


def sparse_decode_one_token(model: Transformer, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs):
    assert input_pos.shape[-1] == 1
    return sample(model.sparse_forward(x, input_pos), **sampling_kwargs)


class DecodeGraph:
    """One decode step recorded as a HIP graph: token and position live in
    static device buffers, a replay computes the next token into `tok` and
    advances `pos`.  `check()` replays it against the eager step."""

    def __init__(self, model: Transformer, batch_size: int, decode_type: str, device):
        self.model, self.decode_type = model, decode_type
        self.tok = torch.zeros((batch_size, 1), dtype=torch.int, device=device)
        self.pos = torch.zeros((1,), dtype=torch.long, device=device)
        self.logits: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None

    def _step(self):
        fwd = self.model.forward if self.decode_type == "dense" else self.model.sparse_forward
        logits = fwd(self.tok, self.pos)
        nxt = torch.argmax(logits[:, -1], dim=-1, keepdim=True).to(torch.int)
        return logits, nxt

    @torch.no_grad()
    def capture(self, tok: torch.Tensor, pos: int) -> None:
        self.tok.copy_(tok)
        self.pos.fill_(pos)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):          # warm the allocator and library handles off the capture
            for _ in range(2):
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        hash_cache.prepare_one_launch_attention(self.tok.device)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits, nxt = self._step()
            self.tok.copy_(nxt)
            self.pos.add_(1)

    @torch.no_grad()
    def check(self, tok: torch.Tensor, pos: int, replays: int = 3) -> dict:
        """Replay the step `replays` times from the same state, with eager work
        and synchronisations in between, and compare every replay with the eager
        step (which rewrites the same cache row, so the state is stationary)."""
        self.tok.copy_(tok)
        self.pos.fill_(pos)
        want_logits, want_next = self._step()
        want_logits = want_logits.float().clone()
        worst, same_token = 0.0, True
        for _ in range(replays):
            self.tok.copy_(tok)
            self.pos.fill_(pos)
            self.graph.replay()
            torch.cuda.synchronize()
            worst = max(worst, float((self.logits.float() - want_logits).abs().max()))
            same_token = same_token and bool(torch.equal(self.tok, want_next))
            _ = (want_logits * 2).sum().item()          # unrelated eager work between replays
        return {"replays": replays, "max_abs_logit_diff": worst, "same_token": same_token}

    def replay(self) -> None:
        self.graph.replay()


@torch.no_grad()
def decode_n_tokens(model: Transformer, cur_token: torch.Tensor, input_pos: torch.Tensor, num_new_tokens: int,
                    callback: Callable = lambda _: _, decode_type: str = "dense",
                    graph: Optional[DecodeGraph] = None, **sampling_kwargs):
    """Greedy decode of `num_new_tokens` tokens (GPT-FAST/generate.py:155-189).
    With `graph` (already captured) each token is one graph replay."""
    new_tokens: List[torch.Tensor] = []
    new_probs: List[torch.Tensor] = []
    if graph is not None:
        graph.tok.copy_(cur_token)
        graph.pos.copy_(input_pos.view(-1)[:1])
        for _ in range(num_new_tokens):
            graph.replay()
            nxt = graph.tok.clone()
            new_tokens.append(nxt)
            callback(nxt)
        input_pos += num_new_tokens
        return new_tokens, new_probs
    one = decode_one_token if decode_type == "dense" else sparse_decode_one_token
    for _ in range(num_new_tokens):
        next_token, next_prob = one(model, cur_token, input_pos, **sampling_kwargs)
        input_pos += 1
        new_tokens.append(next_token.clone())
        new_probs.append(next_prob.clone())
        callback(new_tokens[-1])
        cur_token = new_tokens[-1]
    return new_tokens, new_probs


@torch.no_grad()
def generate(model: Transformer, prompt: torch.Tensor, max_new_tokens: int, *, decode_type: str = "dense",
             callback: Callable = lambda x: x, use_graph: bool = True, check_graph: bool = False,
             **sampling_kwargs) -> Tuple[torch.Tensor, dict]:
    """Prefill `prompt` [B,T], then decode max_new_tokens - 1 more tokens
    greedily (GPT-FAST/generate.py:245-370, without its speculative branch).
    Returns the full sequences and timing statistics."""
    T = prompt.size(1)
    B = prompt.size(0)
    T_new = T + max_new_tokens
    if T_new > model.config.block_size:
        # (GPT-FAST/generate.py:262-268 clamps the cache to block_size and then decodes
        # past its end; here the request is refused before anything is launched)
        raise ValueError(f"prompt ({T}) + max_new_tokens ({max_new_tokens}) = {T_new} exceeds the model's "
                         f"block_size {model.config.block_size}")
    max_seq_length = T_new
    device = prompt.device
    on_gpu = device.type == "cuda"
    model.setup_caches(max_batch_size=B, max_seq_length=max_seq_length)
    if on_gpu and decode_type != "dense":
        warmup_sparse_decode(model, device, T=min(model.max_seq_length, T))
    seq = torch.empty((B, T_new), dtype=prompt.dtype, device=device)
    seq[:, :T] = prompt
    input_pos = torch.arange(0, T, device=device)

    def clock():
        if on_gpu:
            e = torch.cuda.Event(enable_timing=True)
            e.record()
            return e
        return time.perf_counter()

    def elapsed(a, b) -> float:
        if on_gpu:
            torch.cuda.synchronize()
            return a.elapsed_time(b) / 1e3
        return b - a

    if on_gpu:
        torch.cuda.synchronize()
    t0 = clock()
    next_token = prefill(model, prompt, input_pos, decode_type, **sampling_kwargs)
    t1 = clock()
    prefill_time_s = elapsed(t0, t1)
    seq[:, T] = next_token[:, 0]

    graph, graph_report = None, None
    if on_gpu and use_graph and max_new_tokens > 1:
        graph = DecodeGraph(model, B, decode_type, device)
        graph.capture(next_token, T)
        if check_graph:
            graph_report = graph.check(next_token, T)

    input_pos = torch.tensor([T], device=device, dtype=torch.long)
    t2 = clock()
    generated, _ = decode_n_tokens(model, next_token, input_pos, max_new_tokens - 1, callback=callback,
                                   decode_type=decode_type, graph=graph, **sampling_kwargs)
    t3 = clock()
    decode_time_s = elapsed(t2, t3)
    if generated:
        seq[:, T + 1:] = torch.cat(generated, dim=1)
    stats = {
        "prefill_time_s": prefill_time_s,
        "decode_time_s": decode_time_s,
        "decode_only_tokens": B * max(0, max_new_tokens - 1),
        "graph": graph is not None,
        "graph_check": graph_report,
    }
    return seq, stats


def load_random_model(name_or_args, device, precision=torch.bfloat16, seed: int = 1234) -> Transformer:
    """A model of the named geometry with weights ~ N(0, 0.02) and hash planes /
    prototypes ~ N(0, 0.02) (the initialisation GPT-FAST/generate.py:415-422 gives
    the hash buffers), materialised directly on `device`."""
    args = name_or_args if isinstance(name_or_args, ModelArgs) else ModelArgs.from_name(name_or_args)
    with torch.device("meta"):
        model = Transformer(args)
    model = model.to_empty(device=device).to(dtype=precision)
    gen = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for name, p in list(model.named_parameters()) + list(model.named_buffers()):
            if p is None:
                continue
            if name.endswith("norm.weight"):
                p.fill_(1.0)
            else:
                p.normal_(mean=0.0, std=0.02, generator=gen)
    return model.eval()


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description="Greedy decode with dense or SOCKET sparse attention on random weights")
    ap.add_argument("--model", default="Llama-3.1-8B")
    ap.add_argument("--n_layer", type=int, default=None, help="override the number of layers")
    ap.add_argument("--prompt_len", type=int, default=65536)
    ap.add_argument("--max_new_tokens", type=int, default=256)
    ap.add_argument("--batch_size", type=int, default=1)
    ap.add_argument("--decode_type", choices=["dense", "sparse", "both"], default="both")
    ap.add_argument("--no_graph", action="store_true")
    ap.add_argument("--check_graph", action="store_true")
    ap.add_argument("--seed", type=int, default=1234)
    a = ap.parse_args(argv)

    device = torch.device("cuda")
    cfg = ModelArgs.from_name(a.model)
    if a.n_layer is not None:
        cfg.n_layer = a.n_layer
    model = load_random_model(cfg, device, torch.bfloat16, a.seed)
    g = torch.Generator().manual_seed(a.seed)
    prompt = torch.randint(0, cfg.vocab_size, (a.batch_size, a.prompt_len), generator=g).to(device)
    kinds = ["sparse", "dense"] if a.decode_type == "both" else [a.decode_type]
    report = {"model": a.model, "n_layer": cfg.n_layer, "prompt_len": a.prompt_len,
              "max_new_tokens": a.max_new_tokens, "batch_size": a.batch_size}
    outs = {}
    for kind in kinds:
        seq, st = generate(model, prompt, a.max_new_tokens, decode_type=kind, use_graph=not a.no_graph,
                           check_graph=a.check_graph)
        tok_s = st["decode_only_tokens"] / st["decode_time_s"] if st["decode_time_s"] > 0 else float("nan")
        report[kind] = {"decode_tok_s": tok_s, **st}
        outs[kind] = seq[:, a.prompt_len:].cpu()
    if len(outs) == 2:
        same = (outs["sparse"] == outs["dense"]).float().mean().item()
        report["sparse_vs_dense_token_agreement"] = same
    print(json.dumps(report))


if __name__ == "__main__":
    main()
