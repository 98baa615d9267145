"""End-to-end decode and prefill of a Hugging Face decoder with packed linears, next to the same
model with dense fp16 linears of the dequantised weights.

    python -m cobalt_amd.bench_decoder --layers 8            # Mistral-7B block shape, random weights

Decode is timed as HIP-graph replays of one single-token step on a static KV cache (the
protocol of the reference's src/prod/bench.py: steady-state tokens per second at batch 1), so
that the number is the GPU work of a step and not the Python dispatch of its ~40 small kernels
per block.  Prints one JSON line per measurement.  There are no checkpoints or datasets here:
weights are random-initialised and calibration tokens are random ids, which leaves the timing
unaffected and says nothing about accuracy.
"""
from __future__ import annotations

import argparse
import json
import time

import torch


def _decode_tokens_per_s(tr, model, cfg, dev, steps: int, prompt: int, max_len: int) -> float:
    cache = tr.StaticCache(config=cfg, max_cache_len=max_len)
    ids = torch.randint(0, cfg.vocab_size, (1, prompt), device=dev)
    tok = torch.zeros(1, 1, dtype=torch.long, device=dev)
    pos = torch.zeros(1, dtype=torch.long, device=dev)
    with torch.no_grad():
        out = model(ids, past_key_values=cache, cache_position=torch.arange(prompt, device=dev), use_cache=True)
        tok.copy_(out.logits[:, -1:].argmax(-1))
        pos.fill_(prompt)

        def step():
            o = model(tok, past_key_values=cache, cache_position=pos, use_cache=True)
            tok.copy_(o.logits[:, -1:].argmax(-1))
            pos.add_(1)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
    return steps / (time.perf_counter() - t0)


def _prefill_ms(model, cfg, dev, tokens: int, reps: int = 3) -> float:
    ids = torch.randint(0, cfg.vocab_size, (1, tokens), device=dev)
    with torch.no_grad():
        model(ids)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            model(ids)
        torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps * 1e3


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--inter", type=int, default=14336)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--kv-heads", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--sparsity", type=float, default=0.5)
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--prefill", type=int, default=2048)
    a = ap.parse_args(argv)
    import transformers as tr
    from . import model as Mo
    if not torch.cuda.is_available():
        raise SystemExit("bench_decoder needs the GPU: the packed layers have no CPU path")
    dev = "cuda:0"
    cfg = tr.MistralConfig(vocab_size=a.vocab, hidden_size=a.hidden, intermediate_size=a.inter,
                           num_hidden_layers=a.layers, num_attention_heads=a.heads, num_key_value_heads=a.kv_heads,
                           max_position_embeddings=4096, sliding_window=None)
    torch.manual_seed(0)
    model = tr.MistralForCausalLM(cfg).to(dev, torch.float16).eval()
    t0 = time.time()
    calib = torch.randint(0, a.vocab, (4, 256), device=dev)
    rep = Mo.compress_model(model, calib, sparsity=a.sparsity, bits=a.bits, group=a.group, layers_per_pass=2)
    base = dict(layers=a.layers, hidden=a.hidden, inter=a.inter, sparsity=a.sparsity, bits=a.bits, group=a.group,
                bpw=next(iter(rep.values()))["bpw"], data="random weights, random calibration ids",
                compress_s=round(time.time() - t0, 1))
    for name in ("packed", "packed, q|k|v and gate/up fused", "dense fp16 twin"):
        if name.startswith("packed,"):
            Mo.fuse_model(model)
        elif name != "packed":
            model = Mo.dense_twin(model, torch.float16)
        tps = _decode_tokens_per_s(tr, model, cfg, dev, a.steps, 16, 512)
        pms = _prefill_ms(model, cfg, dev, a.prefill)
        print(json.dumps(dict(base, linears=name, decode_tokens_per_s=round(tps, 1),
                              prefill_tokens=a.prefill, prefill_ms=round(pms, 2))), flush=True)


if __name__ == "__main__":
    main()
