"""Measurement helpers shared by ``bench.py`` and ``tools/``: decode latency points (hipGraph-replayed
decode steps timed with HIP events, prefill excluded) and end-to-end generate throughput.

BASELINE.md's protocol: decode tokens/s = B x generated tokens / decode wall time, hipGraph replay,
prefill excluded; prompts of 128 synthetic tokens, max_gen_len 256, B in {1, 8, 32}, greedy.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .engine import DecodeEngine, GenerationConfig


def synthetic_prompts(vocab: int, batch: int, prompt_len: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(3, vocab, (batch, prompt_len), generator=g, dtype=torch.int32)


def decode_latency(model, batch: int, prompt_len: int = 128, gen_len: int = 256, steps: Optional[int] = None,
                   seed: int = 0, barrier=None, do_sample: bool = False) -> Dict[str, float]:
    """Prefill ``batch`` prompts into a ``prompt_len + gen_len`` cache (``prefill_ms``: the second, warm prefill; the
    first autotunes), capture the decode step (every layer, lm_head, sampler, state update), prefill again, then time
    ``steps`` replays of it -- by default every step of a ``gen_len``-token generation (``gen_len - 1`` replays after
    the prefill's first token, cache length from ``prompt_len + 1`` up), so attention is weighted as in a real
    generation (``kv_len_mean`` reports the mean cache length the steps covered; reference generation.py:35:
    max_length = S + max_gen_len). Every rank of a TP group must call this with the same arguments."""
    steps = gen_len - 1 if steps is None else steps
    assert 1 <= steps <= gen_len - 1, "replays must stay inside the cache"
    max_len = prompt_len + gen_len
    eng = DecodeEngine(model, batch, max_len, use_graph=True)
    gc = GenerationConfig(max_length=max_len, do_sample=do_sample, temperature=0.8, top_p=0.95, top_k=50,
                          pad_token_id=0, eos_token_id=-1)
    eng.gc = gc
    prompts = synthetic_prompts(model.config.vocab_size, batch, prompt_len, seed)
    dev = model.device
    eng.prefill(prompts, None)  # cold: autotunes new prefill shapes and grows the workspaces; not timed
    torch.cuda.synchronize(dev)
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    ev0.record()
    eng.prefill(prompts, None)  # warm prefill: ``prefill_ms``
    ev1.record()
    eng._decode_step()  # eager step: sizes the workspaces before capture
    eng.keep_graph = True
    eng._ensure_graph()
    eng._graph.replay()
    torch.cuda.synchronize(dev)
    ttft_ms = ev0.elapsed_time(ev1)
    kernels = graph_kernels(eng._graph)
    eng.prefill(prompts, None)  # back to the first decode position: the timed replays cover the whole window
    torch.cuda.synchronize(dev)
    if barrier is not None:
        barrier()
    ev0.record()
    for _ in range(steps):
        eng._graph.replay()
    ev1.record()
    torch.cuda.synchronize(dev)
    ms = ev0.elapsed_time(ev1) / steps
    model.comm.check()
    del eng
    return {"batch": batch, "decode_ms_per_token": round(ms, 4),
            "decode_tokens_per_sec": round(batch * 1000.0 / ms, 2), "prefill_ms": round(ttft_ms, 3),
            "steps": steps, "kv_len_mean": round(prompt_len + 1 + (steps - 1) / 2, 1),
            # launches of one decode step, counted from the captured graph's kernel nodes (every layer, lm_head,
            # sampler, state update)
            "kernels_per_step": kernels,
            "kernels_per_layer": round(kernels / model.config.num_hidden_layers, 2) if kernels >= 0 else None}


def graph_kernels(graph) -> int:
    """Kernel nodes of a captured torch.cuda.CUDAGraph (hipGraphGetNodes; -1 when the raw graph is unavailable)."""
    from .. import ops
    try:
        return int(ops.ext().graph_kernel_nodes(int(graph.raw_cuda_graph())))
    except (AttributeError, RuntimeError):
        return -1


def time_to_first_token(model, batch: int, prompt_len: int, reps: int = 3, seed: int = 0,
                        barrier=None) -> Dict[str, float]:
    """Prefill of ``batch`` synthetic prompts of ``prompt_len`` tokens up to the first generated token
    (every layer's GEMMs + flash attention + KV-cache writes, last-position lm_head, greedy argmax),
    timed with HIP events after one warm-up prefill (autotune, workspace growth). Median of ``reps``."""
    eng = DecodeEngine(model, batch, prompt_len + 8, use_graph=False)
    gc = GenerationConfig(max_length=prompt_len + 8, do_sample=False, pad_token_id=0, eos_token_id=-1)
    prompts = synthetic_prompts(model.config.vocab_size, batch, prompt_len, seed)
    dev = model.device
    eng.prefill_only(prompts, None, gc)
    torch.cuda.synchronize(dev)
    if barrier is not None:
        barrier()
    times = []
    for _ in range(reps):
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        ev0.record()
        eng.prefill_only(prompts, None, gc)
        ev1.record()
        torch.cuda.synchronize(dev)
        times.append(ev0.elapsed_time(ev1))
    model.comm.check()
    del eng
    ms = sorted(times)[len(times) // 2]
    return {"batch": batch, "prompt_len": prompt_len, "ttft_ms": round(ms, 3),
            "prefill_tokens_per_sec": round(batch * prompt_len * 1000.0 / ms, 1)}


def generate_tokens_per_sec(model, batch: int, prompt_len: int, gen_len: int, gc: GenerationConfig,
                            seed: int = 0, reps: int = 1, barrier=None) -> Dict[str, float]:
    """Whole ``generate`` calls (prefill + every decode step + sampler), output tokens per second."""
    import time
    prompts = synthetic_prompts(model.config.vocab_size, batch, prompt_len, seed)
    dev = model.device
    model.generate(prompts, generation_config=gc)  # warm-up: engine, capture, autotune
    torch.cuda.synchronize(dev)
    if barrier is not None:
        barrier()
    t0 = time.perf_counter()
    for _ in range(reps):
        model.generate(prompts, generation_config=gc)
    torch.cuda.synchronize(dev)
    dt = (time.perf_counter() - t0) / reps
    return {"batch": batch, "ms_per_generate": round(1000 * dt, 2), "tokens_per_sec": round(batch * gen_len / dt, 2)}


def _sclk_levels():
    """(current level line, max level line) of the shader clock from sysfs (pp_dpm_sclk), or (None, None)."""
    import glob
    try:
        for f in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
            lines = [ln.strip() for ln in open(f) if ln.strip()]
            if lines:
                cur = next((ln for ln in lines if ln.endswith("*")), None)
                return cur, lines[-1]
    except OSError:
        pass
    return None, None


def calibration(device) -> Dict[str, object]:
    """Fixed-work probes that tell a slower box from a kernel regression (bench.py ``calibration``):
      * bf16 GEMM TFLOP/s of one fixed 8192^3 shape on this framework's tiled GEMM and on the vendor library
        (torch.mm -> hipBLASLt);
      * ``stream_read_tbps``: a 2 GiB read-only stream through the repo's grid-strided streaming-read kernel
        (norm_embed.hip prefetch_kernel, 16 loads in flight per lane, 4 workgroups per CU); ``stream_read_seq_tbps``:
        the same bytes in the decode kernels' pattern (one contiguous range per wave, stream_probe_kernel) -- the box's
        read roofline, which bench.py divides the streamed bytes by (``hbm_roofline_ms_per_token_box``) beside the fixed
        6.29 TB/s of the guide's copy measurement; ``copy_tbps`` (a torch copy, read + write bytes) is kept beside them;
      * ``sclk_mhz_mfma_probe``: the shader clock measured in-kernel (cycle counter over the constant 100 MHz counter)
        under a dependent-MFMA loop on constant, low-entropy operands -- an upper bound: a GEMM on random data draws
        more power and the chip gives clock back (gate_up at M = 8192 ran at ~1.65 GHz effective under the profiler,
        profiles/r5_pmc_gemm4_vs_hipblaslt_gateup8192.txt); ``sclk_max_level`` from sysfs."""
    from .. import ops
    from ..models.weights import PackedLinear
    out: Dict[str, object] = {}
    n = 8192
    g = torch.Generator(device=device).manual_seed(1)
    x = torch.randn(n, n, device=device, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, n, device=device, generator=g) * 0.02).to(torch.bfloat16)
    pw = PackedLinear.from_dense(w, device)
    y = torch.empty(n, n, device=device, dtype=torch.bfloat16)
    e = ops.ext()

    def timed(fn, iters):
        for _ in range(2):
            fn()
        torch.cuda.synchronize(device)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(iters):
            fn()
        ev1.record()
        torch.cuda.synchronize(device)
        return ev0.elapsed_time(ev1) / iters

    def gemm():
        e.gemm(x, pw.weight, n, n, y, ops.MODE_STORE, False, None, 1, None, -1.0, 0)

    flop = 2.0 * n * n * n
    ms = timed(gemm, 10)
    out["gemm_8192_tflops"] = round(flop / ms / 1e9, 1)
    # the clock under a full matrix load, measured in-kernel (shader cycles / 100 MHz real-time ticks over ~50 ms of
    # dependent MFMA chains on every CU; norm_embed.hip clock_probe_kernel) -- sysfs shows only the DPM request level
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    ticks = torch.zeros(3, dtype=torch.int64, device=device)
    e.clock_probe(200, 4 * cus, ticks)  # warm
    e.clock_probe(1000000, 4 * cus, ticks)
    torch.cuda.synchronize(device)
    cyc, rt = (int(v) for v in ticks[:2].tolist())
    if rt > 0:
        out["sclk_mhz_mfma_probe"] = round(cyc / rt * 100.0, 1)
    cur, top = _sclk_levels()
    if top is not None:
        out["sclk_max_level"] = top
    ms = timed(lambda: torch.mm(x, w.t(), out=y), 10)
    out["hipblaslt_8192_tflops"] = round(flop / ms / 1e9, 1)
    del x, w, pw, y
    src = torch.empty(1 << 29, dtype=torch.float32, device=device).fill_(1.0)  # 2 GiB
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    ms = timed(lambda: ext_prefetch(e, src, 4 * cus), 5)  # (cus: set above)
    out["stream_read_tbps"] = round(src.numel() * 4 / ms / 1e9, 2)
    # the decode kernels' own pattern: each wave one contiguous range, 1 KiB per instruction (norm_embed.hip
    # stream_probe_kernel; 8 workgroups per CU) -- the read rate a decode weight / KV stream can reach on this box
    ms = timed(lambda: ext_prefetch(e, src, -8 * cus), 5)
    out["stream_read_seq_tbps"] = round(src.numel() * 4 / ms / 1e9, 2)
    dst = torch.empty_like(src)
    ms = timed(lambda: dst.copy_(src), 5)
    out["copy_tbps"] = round(2 * src.numel() * 4 / ms / 1e9, 2)
    del src, dst
    torch.cuda.empty_cache()
    return out


def ext_prefetch(e, t: torch.Tensor, grid: int) -> None:
    e.prefetch(t, int(grid))


# ---------------------------------------------------------------------------------------------------------------
# Hybrid (Zavevik) family beside LLaMA at equal layer sizes
# ---------------------------------------------------------------------------------------------------------------
HYBRID_SIZES = {
    # name: width, heads, kv heads, head dim, dense FFN width (= the experts' active width), layers, vocab
    "2k": dict(width=2048, heads=16, kv_heads=4, head_dim=128, ffn=5632, layers=4, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, layers=4, vocab=32000),
}


def zavevik_like(width: int, heads: int, kv_heads: int, head_dim: int, ffn: int, layers: int, vocab: int,
                 experts: int = 8, top: int = 2):
    """A Zavevik config whose layers have a LLaMA layer's sizes: delta, attention, attention on the previous layer's
    keys, delta, ...; ``experts`` experts of width ``ffn / top`` (the active width equals the dense FFN's)."""
    from ..config import ZavevikConfig
    att = dict(heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, scale=head_dim ** -0.5, softcap=50.0,
               bias_max=4096, q_temp={"coef": 0.1, "every": 256})
    dl = dict(heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, conv=4)
    mlp = {"kind": "moe", "expert": {"ff": ffn // top}, "router": {"experts": experts, "top": top}}
    ls = []
    for i in range(layers):
        if i % 4 in (0, 3):
            ls.append({"type": "delta", "mixer": dict(dl), "mlp": mlp})
        elif i % 4 == 1:
            ls.append({"type": "attention", "mixer": dict(att), "mlp": mlp})
        else:
            ls.append({"type": "attention", "mixer": dict(att, kv_from=i - 1), "mlp": mlp})
    return ZavevikConfig.from_dict({"architecture": "Zavevik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
                                    "token_side": {"dim": 64}, "layers": ls})


def zasevik_like(width: int, heads: int, kv_heads: int, head_dim: int, ffn: int, layers: int, vocab: int,
                 kv_rank: int = 512, experts: int = 8, top: int = 2):
    """A Zasevik config whose layers have a LLaMA layer's sizes: ``heads`` heads of ``head_dim`` over a latent of
    ``kv_rank``; feed-forwards alternate between dense (width ``ffn``) and routed (``top`` of ``experts`` experts of
    width ``ffn / 4`` plus a shared expert of ``ffn / 2``: the active width equals the dense FFN's at top 2).
    ``kv_heads`` has no counterpart (one latent serves every head)."""
    from ..config import ZasevikConfig
    mix = dict(heads=heads, dim=head_dim, vdim=head_dim, kv_rank=kv_rank, scale=head_dim ** -0.5)
    moe = {"kind": "moe", "expert": {"ff": ffn // 4, "limit": 7.0}, "router": {"experts": experts, "top": top},
           "shared": {"ff": ffn // 2, "limit": 7.0}}
    ls = [{"type": "latent_attention", "mixer": dict(mix), "mlp": moe if i % 2 else {"kind": "dense", "ff": ffn}}
          for i in range(layers)]
    return ZasevikConfig.from_dict({"architecture": "Zasevik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
                                    "embedding": {"scale": width ** 0.5}, "layers": ls})


def besulix_like(width: int, heads: int, kv_heads: int, head_dim: int, ffn: int, layers: int, vocab: int,
                 chunk: int = 1024, timemix_dim: int = 64):
    """A Besulix config whose layers have a LLaMA layer's sizes: parallel layers (``heads`` / ``kv_heads`` attention
    heads of ``head_dim``, half of each q / k head rotated, blocks of ``chunk`` positions, beside ``width /
    timemix_dim`` time-mix heads of ``timemix_dim``; dense feed-forward of ``ffn``) alternating with matrix-memory
    layers (``heads`` heads of ``head_dim`` keys and values, no feed-forward)."""
    from ..config import BesulixConfig
    left = dict(heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, scale=head_dim ** -0.5,
                rot={"base": 1e4, "dims": head_dim // 2}, mask={"size": chunk})
    par = {"left": left, "right": {"heads": max(1, width // timemix_dim), "dim": timemix_dim}, "left_scale": 0.7,
           "right_scale": 0.7}
    mls = dict(heads=heads, dim=head_dim, vdim=head_dim, gate_cap=15.0)
    ls = [{"type": "mlstm", "mixer": dict(mls), "mlp": None} if i % 2 else
          {"type": "parallel", "mixer": par, "mlp": {"kind": "dense", "ff": ffn, "limit": 7.0}} for i in range(layers)]
    return BesulixConfig.from_dict({"architecture": "Besulix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
                                    "logit_softcap": 30.0, "layers": ls})


def zifisun_like(width: int, heads: int, kv_heads: int, head_dim: int, ffn: int, layers: int, vocab: int,
                 kv_rank: int = 448, window: int = 1024, experts: int = 8, identity: int = 2, top: int = 2,
                 streams: int = 2):
    """A Zifisun config whose layers have a LLaMA layer's sizes: latent-attention layers (``heads`` heads whose keys are
    ``head_dim / 2`` plain + ``head_dim / 2`` rotated numbers, values of ``head_dim``, a latent of ``kv_rank`` so that a
    cache row is ``kv_rank + head_dim / 2`` wide, a query latent of ``3 kv_rank / 2``) alternating with attention layers
    (``heads`` / ``kv_heads`` heads of ``head_dim``, the first 64 keys kept), windows of ``window``; every layer with a
    mixture of ``experts`` experts of ``ffn / 4`` plus ``identity`` identity experts in 5 groups of which 3 are kept,
    ``top`` per token, and a shared expert of ``ffn / 2`` (the active width of the dense FFN at top 2); ``streams``
    residual streams."""
    from ..config import ZifisunConfig
    half = head_dim // 2
    lat = dict(heads=heads, dim=half, rot_dim=half, vdim=head_dim, kv_rank=kv_rank, q_rank=kv_rank * 3 // 2,
               scale=head_dim ** -0.5, rot={"base": 1e4, "dims": half}, mask={"size": window})
    att = dict(heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, scale=head_dim ** -0.5,
               mask={"size": window, "keep_first": 64})
    total = experts + identity
    groups = 5 if total % 5 == 0 else 1
    moe = {"kind": "moe", "expert": {"ff": ffn // 4},
           "router": {"experts": experts, "identity": identity, "top": top,
                      "groups": {"count": groups, "keep": min(3, groups)}},
           "shared": {"ff": ffn // 2}}
    ls = [{"type": "attention", "mixer": dict(att), "mlp": moe} if i % 2 else
          {"type": "latent_attention", "mixer": dict(lat), "mlp": moe} for i in range(layers)]
    return ZifisunConfig.from_dict({"architecture": "Zifisun", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
                                    "streams": streams, "layers": ls})


def hybrid_compare(device, sizes=("2k", "4k"), prompt_len: int = 2048, gen_len: int = 64, batches=(1, 8),
                   families=("zavevik", "llama"), progress=lambda m: None) -> Dict[str, object]:
    """Prefill and decode throughput of the layer-list families (Zavevik, Zasevik, Besulix, Zifisun) beside LLaMA at equal layer sizes
    (random weights, bf16, synthetic ids), all through the decode engine: ``prefill_tokens_per_sec`` of one warm ``prompt_len``-token prompt per row
    and hipGraph-replayed ``decode_ms_per_token`` over ``gen_len`` steps behind it."""
    from ..config import LLaMAConfig
    from ..models.llama import LLaMAForCausalLM
    from ..models.zavevik import ZavevikForCausalLM
    out: Dict[str, object] = {"prompt_len": prompt_len, "gen_len": gen_len, "dtype": "bf16",
                              "data": "synthetic token ids, random-init weights"}
    for name in sizes:
        sz = HYBRID_SIZES[name]
        row: Dict[str, object] = {"size": sz}
        for family in families:
            if family == "zavevik":
                model = ZavevikForCausalLM(zavevik_like(**sz), device=device, dtype=torch.bfloat16, seed=1)
            elif family == "zasevik":
                from ..models.zasevik import ZasevikForCausalLM
                model = ZasevikForCausalLM(zasevik_like(**sz), device=device, dtype=torch.bfloat16, seed=1)
            elif family == "besulix":
                from ..models.besulix import BesulixForCausalLM
                model = BesulixForCausalLM(besulix_like(**sz), device=device, dtype=torch.bfloat16, seed=1)
            elif family == "zifisun":
                from ..models.zifisun import ZifisunForCausalLM
                model = ZifisunForCausalLM(zifisun_like(**sz), device=device, dtype=torch.bfloat16, seed=1)
            else:
                cfg = LLaMAConfig(vocab_size=sz["vocab"], hidden_size=sz["width"], intermediate_size=sz["ffn"],
                                  num_hidden_layers=sz["layers"], num_attention_heads=sz["heads"],
                                  num_key_value_heads=sz["kv_heads"], max_sequence_length=prompt_len + gen_len)
                model = LLaMAForCausalLM(cfg, device=device, _do_init=False).init_random(seed=1)
            pts = []
            for b in batches:
                r = decode_latency(model, b, prompt_len=prompt_len, gen_len=gen_len)
                r["prefill_tokens_per_sec"] = round(b * prompt_len * 1000.0 / r["prefill_ms"], 1)
                pts.append(r)
                progress(f"{name} {family} B={b}: prefill {r['prefill_ms']} ms, decode {r['decode_ms_per_token']} ms")
            row[family] = {"weight_gb": round(model.weight_bytes() / 1e9, 3), "points": pts}
            del model
            torch.cuda.empty_cache()
        out[name] = row
    return out
