"""Serving throughput of a Lenitar configuration beside the closest existing model (the routed-expert
transformer: softmax attention + top-k SwiGLU experts) at equal width, depth, heads and experts, and of
a Dumalix configuration beside the dense transformer (grouped-query softmax attention + SwiGLU) at equal
width, layer runs, heads, kv heads and feed-forward size, and of a Malinex configuration beside Lenitar (the
closest existing model: recurrent-state layers among attention layers, routed experts, an fp32 residual
stream) at equal width, depth, heads, experts and expert size, and of a Pamazen configuration beside Malinex (the
closest existing model: grouped-query attention over paged rows beside a decayed matrix memory in state slots,
softmax-routed experts with a shared one, an fp32 residual stream) at equal width, depth, heads, kv heads, experts
and expert size.

Both run through the same engine calls: one prompt portion per sequence (``InferenceEngine.prefill``)
and then one-token decode steps of the whole batch (``InferenceEngine.decode``); random weights,
synthetic tokens.  Reported: prefill tokens/s (one prompt of ``prompt`` tokens) and decode tokens/s
(``batch`` sequences at that context).
"""

from __future__ import annotations

import time
from typing import Dict, List

import torch

SIZES = {
    "tiny": dict(width=128, layers=4, heads=4, experts=4, top=2, ff=64, window=32, prompt=64, batch=2),
    # name: width, layers, heads, experts, top, expert ff, window, prompt, decode batch
    "small": dict(width=1024, layers=4, heads=8, experts=8, top=2, ff=512, window=512, prompt=2048, batch=16),
    "medium": dict(width=2048, layers=4, heads=16, experts=8, top=2, ff=1024, window=1024, prompt=2048, batch=16),
    "large": dict(width=4096, layers=4, heads=32, experts=8, top=2, ff=2048, window=1024, prompt=4096, batch=16),
}


# Dumalix: width, layers (every third is chunked grouped-query attention, the others latent attention),
# loop (start, stop, times), heads of 128, kv heads, feed-forward, chunk, prompt, decode batch
DUMALIX_SIZES = {
    "tiny": dict(width=128, layers=3, loop=(1, 2, 2), heads=4, kv_heads=2, head_dim=32, ff=192, chunk=32, prompt=64, batch=2),
    "small": dict(width=1024, layers=6, loop=(2, 5, 2), heads=8, kv_heads=2, head_dim=128, ff=3072, chunk=1024, prompt=2048, batch=16),
    "medium": dict(width=2048, layers=6, loop=(2, 5, 2), heads=16, kv_heads=4, head_dim=128, ff=6144, chunk=1024, prompt=2048, batch=16),
    "large": dict(width=4096, layers=6, loop=(2, 5, 2), heads=32, kv_heads=8, head_dim=128, ff=12288, chunk=2048, prompt=4096, batch=16),
}


# Malinex: width, layers (every third is sigmoid attention, the others gated linear attention), heads of
# ``head_dim`` (gated linear attention: keys of half that), kv heads, routed experts + one shared, prompt, decode batch
MALINEX_SIZES = {
    "tiny": dict(width=128, layers=3, heads=4, kv_heads=2, head_dim=32, experts=4, top=2, ff=64, prompt=64, batch=2),
    "small": dict(width=1024, layers=6, heads=8, kv_heads=2, head_dim=128, experts=8, top=2, ff=512, prompt=2048, batch=16),
    "medium": dict(width=2048, layers=6, heads=16, kv_heads=4, head_dim=128, experts=8, top=2, ff=1024, prompt=2048, batch=16),
}  # (no width 4096: Lenitar's latent rank of width / 4 is then beyond its attention kernels)


# Pamazen: width, layers (every third is the parallel pair of windowed attention and delta-rule memory, the others
# rotary attention), heads of ``head_dim`` (delta rule: heads of half that), kv heads, routed gated experts + one shared,
# four residual streams, window, prompt, decode batch
PAMAZEN_SIZES = {
    "tiny": dict(width=128, layers=3, heads=4, kv_heads=2, head_dim=32, experts=4, top=2, ff=64, window=32, prompt=64, batch=2),
    "small": dict(width=1024, layers=6, heads=8, kv_heads=2, head_dim=128, experts=8, top=2, ff=512, window=1024, prompt=2048, batch=16),
    "medium": dict(width=2048, layers=6, heads=16, kv_heads=4, head_dim=128, experts=8, top=2, ff=1024, window=1024, prompt=2048, batch=16),
    "large": dict(width=4096, layers=6, heads=32, kv_heads=8, head_dim=128, experts=8, top=2, ff=2048, window=1024, prompt=4096, batch=16),
}


def _configs_pamazen(s: Dict):
    from llmctl.models.malinex import malinex_template
    from llmctl.models.pamazen import pamazen_template

    pa = pamazen_template(width=s["width"], layers=s["layers"], heads=s["heads"], kv_heads=s["kv_heads"], vocab=32000, every=3,
                          experts=s["experts"], top=s["top"], expert_ff=s["ff"], head_dim=s["head_dim"], streams=4, window=s["window"])
    pa.max_position_embeddings = s["prompt"] + 256
    ma = malinex_template(width=s["width"], layers=s["layers"], heads=s["heads"], kv_heads=s["kv_heads"], vocab=32000, every=3,
                          experts=s["experts"], top=s["top"], expert_ff=s["ff"], head_dim=s["head_dim"],
                          max_positions=s["prompt"] + 256)
    return pa, ma


def _configs_malinex(s: Dict):
    from llmctl.models.lenitar import lenitar_template
    from llmctl.models.malinex import malinex_template

    ma = malinex_template(width=s["width"], layers=s["layers"], heads=s["heads"], kv_heads=s["kv_heads"], vocab=32000, every=3,
                          experts=s["experts"], top=s["top"], expert_ff=s["ff"], head_dim=s["head_dim"],
                          max_positions=s["prompt"] + 256)
    le = lenitar_template(width=s["width"], layers=s["layers"], heads=s["heads"], vocab=32000, every=3, experts=s["experts"],
                          top=s["top"], groups=2, keep=1, ff=s["ff"], window=s["prompt"])
    le.max_position_embeddings = s["prompt"] + 256
    return ma, le


def _configs_dumalix(s: Dict):
    from llmctl.models.config import ModelConfig
    from llmctl.models.dumalix import dumalix_template

    du = dumalix_template(width=s["width"], layers=s["layers"], heads=s["heads"], kv_heads=s["kv_heads"], vocab=32000, every=3,
                          ff=s["ff"], chunk=s["chunk"], taps=4, loop=s["loop"], head_dim=s["head_dim"])
    du.max_position_embeddings = s["prompt"] + 256
    runs = len(du.runs())
    tr = ModelConfig(name=f"dense-w{s['width']}-l{runs}", layers=runs, hidden=s["width"], ffn=s["ff"], heads=s["heads"],
                     kv_heads=s["kv_heads"], vocab_size=32000, max_position_embeddings=s["prompt"] + 256)
    return du, tr


def _configs(s: Dict):
    from llmctl.models.config import ModelConfig
    from llmctl.models.lenitar import lenitar_template

    hy = lenitar_template(width=s["width"], layers=s["layers"], heads=s["heads"], vocab=32000, every=4,
                          experts=s["experts"], top=s["top"], groups=2, keep=1, ff=s["ff"], window=s["window"])
    hy.max_position_embeddings = s["prompt"] + 256
    tr = ModelConfig(name=f"moe-w{s['width']}-l{s['layers']}", layers=s["layers"], hidden=s["width"], ffn=s["ff"],
                     heads=s["heads"], vocab_size=32000, max_position_embeddings=s["prompt"] + 256,
                     num_experts=s["experts"], experts_per_token=s["top"], moe_ffn=s["ff"])
    return hy, tr


def _engine(cfg, device, prompt, batch):
    import json
    import tempfile
    from pathlib import Path

    from llmctl.serve.engine import InferenceEngine

    d = Path(tempfile.mkdtemp(prefix="llmctl_bench_"))
    (d / "m.json").write_text(json.dumps(cfg.to_dict()))
    bs = 16
    blocks = (batch + 1) * ((prompt + 256 + bs - 1) // bs)
    return InferenceEngine(str(d / "m.json"), device=device, max_batch_size=batch, max_batch_tokens=1 << 30,
                           max_model_len=prompt + 256, block_size=bs, num_kv_blocks=blocks, use_graphs=False,
                           prefix_caching=False)


def _measure(eng, prompt: int, batch: int, steps: int, warmup: int) -> Dict[str, float]:
    from llmctl.serve.scheduler import PrefillChunk

    dev = eng.device
    g = torch.Generator().manual_seed(0)
    V = eng.cfg.vocab_size

    def sync():
        if dev.type == "cuda":
            torch.cuda.synchronize()

    # prefill: one prompt per call
    times = []
    for i in range(warmup + steps):
        seq = eng.open_sequence(torch.randint(0, V, (prompt,), generator=g).tolist())
        sync()
        t0 = time.perf_counter()
        eng.prefill([PrefillChunk(seq, 0, prompt)])
        sync()
        times.append(time.perf_counter() - t0)
        eng.scheduler.computed(seq, prompt)
        eng.scheduler.finish(seq, "stop")
    pre = sorted(times[warmup:])[len(times[warmup:]) // 2]
    # decode: ``batch`` sequences at context ``prompt``
    seqs = [eng.open_sequence(torch.randint(0, V, (prompt,), generator=g).tolist()) for _ in range(batch)]
    for s in seqs:
        eng.prefill([PrefillChunk(s, 0, prompt)])
        eng.scheduler.computed(s, prompt)
    times = []
    for i in range(warmup + steps):
        for s in seqs:
            eng.scheduler.extend(s, [int(torch.randint(0, V, (1,), generator=g))])
            s._decode_slot = int(eng.kv.slots(s.seq_id, s.num_tokens - 1, 1)[0])
        sync()
        t0 = time.perf_counter()
        eng.decode(seqs)
        sync()
        times.append(time.perf_counter() - t0)
        for s in seqs:
            eng.scheduler.computed(s, 1)
    dec = sorted(times[warmup:])[len(times[warmup:]) // 2]
    for s in seqs:
        eng.scheduler.finish(s, "stop")
    return {"prefill_ms": round(pre * 1e3, 3), "prefill_tok_s": round(prompt / pre, 1),
            "decode_ms": round(dec * 1e3, 3), "decode_tok_s": round(batch / dec, 1)}


def run(sizes: List[str], device: str = "auto", steps: int = 5, warmup: int = 2, family: str = "lenitar") -> List[Dict]:
    out = []
    for name in sizes:
        if family == "pamazen":
            s = PAMAZEN_SIZES[name]
            hy, tr = _configs_pamazen(s)
            row = {"size": name, **s}
            pair = (("pamazen", hy), ("malinex", tr))
        elif family == "malinex":
            s = MALINEX_SIZES[name]
            hy, tr = _configs_malinex(s)
            row = {"size": name, **s}
            pair = (("malinex", hy), ("lenitar", tr))
        elif family == "dumalix":
            s = DUMALIX_SIZES[name]
            hy, tr = _configs_dumalix(s)
            row = {"size": name, **s, "layer_runs": len(hy.runs())}
            pair = (("dumalix", hy), ("dense_transformer", tr))
        else:
            s = SIZES[name]
            hy, tr = _configs(s)
            row = {"size": name, **{k: s[k] for k in ("width", "layers", "heads", "experts", "top", "ff", "window", "prompt", "batch")}}
            pair = (("lenitar", hy), ("moe_transformer", tr))
        for label, cfg in pair:
            eng = _engine(cfg, device, s["prompt"], s["batch"])
            row[label] = _measure(eng, s["prompt"], s["batch"], steps, warmup)
            row[label]["params_m"] = round(sum(p.numel() for p in eng.model.parameters()) / 1e6, 1)
            eng.close()
        out.append(row)
    return out
