"""Besulix through the framework (model, cache, stepper, engine) against the plain float64 oracle
(tests/oracle_besulix.py), on the CPU op path and, marked gpu, on the HIP kernels. Small configurations built here:
sizes off every tile grid, unequal key / value widths, rotary dims below and equal to the head size, block lengths that
are not multiples of any kernel's tile, one head and many, key heads equal to and fewer than query heads, layers in
several orders with and without feed-forwards."""
import math

import numpy as np
import pytest
import torch

import oracle_besulix as ob
from jax_llama_amd.config import BesulixConfig
from jax_llama_amd.models.besulix import GATE_ALPHA, BesulixForCausalLM, random_state_dict
from jax_llama_amd.models.kv_cache import HybridCache
from jax_llama_amd.models.mixers import (GatedDenseFF, MatrixLSTM, RotaryChunkAttention, SideBySide, StepContext,
                                         TimeMix)
from jax_llama_amd.ops import hybrid as hy
from jax_llama_amd.runtime.engine import GenerationConfig
from jax_llama_amd.runtime.stepper import SequenceStepper

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32, BF16 = torch.float32, torch.bfloat16


def _left(heads, kv, dim, vdim, rot, chunk, scale=0.3, base=50.0):
    return dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, rot={"base": base, "dims": rot},
                mask={"size": chunk})


def _par(left, r_heads, r_dim, ls=0.7, rs=1.3):
    return {"left": left, "right": {"heads": r_heads, "dim": r_dim}, "left_scale": ls, "right_scale": rs}


def _mls(heads, dim, vdim, cap):
    return dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap)


def _ff(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def cfg_full():
    return {"architecture": "Besulix", "vocab": 61, "width": 48, "norm": {"eps": 1e-6}, "logit_softcap": 2.0,
            "layers": [
                {"type": "parallel", "mixer": _par(_left(4, 2, 12, 8, 6, 7), 3, 8), "mlp": _ff(40, 0.8)},
                {"type": "mlstm", "mixer": _mls(3, 8, 12, 4.0), "mlp": None},
                {"type": "mlstm", "mixer": _mls(2, 20, 6, 9.0), "mlp": _ff(24, 2.5)},
                {"type": "parallel", "mixer": _par(_left(6, 3, 8, 10, 8, 16, 0.4, 1e4), 2, 24, 1.1, 0.4), "mlp": None},
            ]}


def cfg_bare():
    """One head everywhere, as many key heads as query heads, every number of a head rotated, equal key and value
    sizes, a block longer than any test sequence, unit mixing weights, a mixer-only stack ending in a feed-forward."""
    return {"architecture": "Besulix", "vocab": 37, "width": 40, "norm": {"eps": 1e-5}, "logit_softcap": 30.0,
            "layers": [
                {"type": "mlstm", "mixer": _mls(1, 40, 40, 15.0), "mlp": None},
                {"type": "parallel", "mixer": _par(_left(1, 1, 16, 16, 16, 1000, 0.25), 1, 16, 1.0, 1.0), "mlp": _ff(56, 7.0)},
            ]}


def cfg_odd():
    """Sizes that are multiples of nothing a kernel loads at once: width 50, vocab 77, heads of 10 / 6 / 14 numbers,
    three of everything, a block of three positions, a feed-forward of 30."""
    return {"architecture": "Besulix", "vocab": 77, "width": 50, "norm": {"eps": 1e-5}, "logit_softcap": 3.0,
            "layers": [
                {"type": "mlstm", "mixer": _mls(3, 10, 14, 2.0), "mlp": _ff(30, 1.0)},
                {"type": "parallel", "mixer": _par(_left(3, 1, 10, 6, 4, 3, 0.31, 7.0), 3, 10, 0.9, 1.1), "mlp": None},
                {"type": "parallel", "mixer": _par(_left(9, 3, 6, 14, 6, 11, 0.5, 300.0), 5, 6, 0.3, 2.0), "mlp": _ff(18, 5.0)},
            ]}


def build(cfg, device, dtype=F32, seed=0, edit=None, decay_rank=5):
    config = BesulixConfig.from_dict(cfg)
    sd = random_state_dict(config, seed=seed, decay_rank=decay_rank)
    for k in list(sd):
        if k.endswith("mlp.gate") or k.endswith("mlp.up"):  # pre-activations on both sides of the clamps
            sd[k] = (sd[k].float() * 2.0).to(BF16)
    if edit:
        edit(sd)
    model = BesulixForCausalLM(config, device=device, dtype=dtype, _do_init=False).load_state_dict(sd)
    return model, sd


def toks(n, vocab, seed=1):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got, ref):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    d = got - ref
    return float(np.sqrt(np.mean(d * d)) / np.sqrt(np.mean(ref * ref)))


def tol(device, dtype=F32):
    return 3e-2 if dtype == BF16 else 2e-5


def run_portions(model, tokens, portions, rid="r", stepper=None, max_tokens=None):
    """Logits of every position through the stepper, the prompt cut into ``portions``."""
    st = stepper or SequenceStepper(model, max_tokens or len(tokens))
    out, at = [], 0
    for n in portions:
        out.append(st.feed(rid, tokens[at:at + n], list(range(n))).float().cpu())
        at += n
    assert at == len(tokens)
    st.end(rid)
    return torch.cat(out).numpy()


def run_mixer(mixer, cache, h, portions, device):
    """A mixer block on hand-made inputs ``h [t, D]`` in portions, through the cache."""
    outs, s0 = [], 0
    for s in portions:
        ids = torch.zeros(s, dtype=torch.int32, device=device)
        pos = torch.arange(s0, s0 + s, dtype=torch.int32, device=device)
        outs.append(mixer(h[s0:s0 + s].to(device).contiguous(), StepContext(ids, pos, 1, s, cache, s0)).cpu())
        s0 += s
    assert s0 == h.shape[0]
    return torch.cat(outs).numpy()


# ---------------------------------------------------------------------------------------------- configuration
def test_config_round_trip():
    c = BesulixConfig.from_dict(cfg_full())
    assert BesulixConfig.from_dict(c.to_dict()) == c and c.num_hidden_layers == 4 and c.logit_softcap == 2.0
    assert c.layers[1].mlp is None and c.layers[2].mlp.ff == 24 and c.layers[2].mlp.limit == 2.5
    assert c.layers[0].mixer.left.chunk == 7 and c.layers[0].mixer.left.rot_dims == 6 and c.layers[0].mixer.right.dim == 8
    assert c.layers[3].mixer.left_scale == 1.1 and c.layers[1].mixer.gate_cap == 4.0
    for breakage in (lambda d: d["layers"][0].__setitem__("type", "delta"),
                     lambda d: d["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 14),   # more than dim
                     lambda d: d["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3),       # 4 % 3
                     lambda d: d["layers"][0]["mixer"]["left"]["mask"].__setitem__("size", 0),
                     lambda d: d["layers"][0]["mlp"].__setitem__("kind", "moe")):
        bad = cfg_full()
        breakage(bad)
        with pytest.raises(ValueError):
            BesulixConfig.from_dict(bad)


# ---------------------------------------------------------------------------------------------- mechanisms alone
def _attn_weights(g, mc, d):
    r = lambda *s, sc: torch.randn(*s, generator=g) * sc  # noqa: E731
    nh, kv, dim, vdim = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    return {"m.q": r(nh * dim, d, sc=0.4), "m.q.b": r(nh * dim, sc=0.3), "m.k": r(kv * dim, d, sc=0.4),
            "m.k.b": r(kv * dim, sc=0.3), "m.v": r(kv * vdim, d, sc=0.4), "m.v.b": r(kv * vdim, sc=0.3),
            "m.temp": torch.rand(nh, generator=g) + 0.5, "m.sink": r(nh, sc=1.5), "m.o": r(d, nh * vdim, sc=0.2)}


def _attn_mixer(w, mc, t, device, dtype=F32, value_turn=True):
    cache = HybridCache([("kv", mc["kv_heads"], mc["dim"], mc["vdim"])], 1, t, device, dtype)
    mixer = RotaryChunkAttention(
        0, mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"], mc["scale"],
        torch.cat([w["m.q"], w["m.k"], w["m.v"]]).to(device, dtype), torch.cat([w["m.q.b"], w["m.k.b"], w["m.v.b"]]).to(device),
        hy.rotary_freqs(mc["rot"]["base"], mc["rot"]["dims"], device),
        hy.rotary_freqs(mc["rot"]["base"], mc["vdim"], device) if value_turn else None, w["m.temp"].to(device),
        w["m.sink"].to(device), mc["mask"]["size"], w["m.o"].to(device, dtype))
    return mixer, cache


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,kv,dim,vdim,rot,chunk", [(4, 2, 12, 8, 6, 7), (3, 3, 16, 16, 16, 5), (2, 1, 8, 40, 4, 64),
                                                         (6, 2, 24, 70, 0, 33), (1, 1, 72, 6, 72, 2), (70, 35, 8, 4, 2, 1)])
def test_chunked_attention_mechanism(device, heads, kv, dim, vdim, rot, chunk):
    """One attention sublayer against the oracle, in portions that start and end inside blocks and include single
    tokens: biases, partial / full / no rotation of q and k, rotated values, temperatures, sinks, blocks of 1 to more
    than the sequence."""
    mc = _left(heads, kv, dim, vdim, rot, chunk, scale=0.37, base=23.0)
    t, d = 41, 48
    g = torch.Generator().manual_seed(3)
    w = _attn_weights(g, mc, d)
    h = torch.randn(t, d, generator=g)
    ref = ob.chunked_sink_attention(w, "m.", mc, h.double().numpy())
    for portions in ([41], [11, 1, 2, 19, 1, 1, 6], [1] * 41):
        mixer, cache = _attn_mixer(w, mc, t, device)
        assert err(run_mixer(mixer, cache, h, portions, device), ref) < 2e-5, portions


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("heads,kv,dim,vdim,rot,chunk", [(4, 2, 64, 64, 32, 48), (2, 1, 128, 64, 128, 100),
                                                         (3, 3, 64, 128, 16, 37), (2, 2, 128, 128, 64, 1000)])
def test_attention_at_the_mfma_head_sizes(device, dtype, heads, kv, dim, vdim, rot, chunk):
    """Head sizes the flash prefill and the fast decode kernels take (bf16 caches), blocks that end inside a 32-key
    tile and inside a wave's 32 queries, portions that start at unaligned slots; both number formats."""
    mc = _left(heads, kv, dim, vdim, rot, chunk, scale=dim ** -0.5, base=1e4)
    t, d = 150, 96
    g = torch.Generator().manual_seed(9)
    w = {k: v.to(BF16).float() for k, v in _attn_weights(g, mc, d).items()}
    h = torch.randn(t, d, generator=g).to(BF16).float()
    ref = ob.chunked_sink_attention(w, "m.", mc, h.double().numpy())
    for portions in ([150], [100, 2, 47, 1], [70] + [1] * 80):
        mixer, cache = _attn_mixer(w, mc, t, device, dtype)
        assert err(run_mixer(mixer, cache, h, portions, device), ref) < (3e-2 if dtype == BF16 else 2e-5), portions


def _aim_query(w, mc, h, qi, kj, strength):
    """Set input ``h[qi]`` so that head 0's rotated query at position ``qi`` points along head 0's rotated key of
    position ``kj``, while the token's own key (head 0 of the keys) is zero, so that a strong query is not also a strong
    key for later ones: the solution of ``W_q[head 0] h + b_q = turn^-1(strength * k / |k|)``, ``W_k[head 0] h + b_k = 0``."""
    dim, rd, base = mc["dim"], mc["rot"]["dims"], mc["rot"]["base"]
    hn = h.double().numpy()
    k = ob.turn((hn[kj] @ w["m.k"].double().numpy().T + w["m.k.b"].double().numpy())[:dim], kj, base, rd)
    target = ob.turn(strength * k / np.linalg.norm(k), -qi, base, rd) - w["m.q.b"].double().numpy()[:dim]
    lhs = np.concatenate([w["m.q"].double().numpy()[:dim], w["m.k"].double().numpy()[:dim]])
    sol = np.linalg.lstsq(lhs, np.concatenate([target, -w["m.k.b"].double().numpy()[:dim]]), rcond=None)[0]
    h[qi] = torch.tensor(sol, dtype=torch.float32).to(BF16).float()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_block_edges_far_keys_and_the_sink_decide(device, dtype):
    """Inputs made so that single keys decide head 0: the first key of a query's block (just inside), the key one
    before it (just outside: it must count for nothing, although the query points straight at it), a far key 160
    positions back in a long block; each once inside a prompt portion and once decoded alone. Head 1's sink takes
    nearly all of that head's weight. A block edge off by one, a lost key or a sink left out moves these rows by far
    more than the tolerance."""
    chunk, t, d = 180, 400, 48
    mc = _left(2, 1, 16, 24, 8, chunk, scale=0.5, base=100.0)
    g = torch.Generator().manual_seed(7)
    w = {k: v.to(BF16).float() for k, v in _attn_weights(g, mc, d).items()}
    w["m.sink"] = torch.tensor([-1.0, 30.0])
    w["m.temp"] = torch.tensor([1.25, 0.75])
    h = (torch.randn(t, d, generator=g) * 0.3).to(BF16).float()
    inside = {(210, 180), (358, 180), (170, 10), (178, 0), (399, 360)}   # (query, key it points at): visible
    outside = {(183, 179), (340, 179), (361, 359), (398, 359)}          # the key just before the query's block
    for qi, kj in sorted(inside | outside):
        _aim_query(w, mc, h, qi, kj, 16.0)
    ref, pw = ob.chunked_sink_attention(w, "m.", mc, h.double().numpy(), return_weights=True)
    for qi, kj in inside:
        assert pw[0, qi, kj] > 0.9, (qi, kj, pw[0, qi, kj])
    for qi, kj in outside:
        assert pw[0, qi, kj] == 0.0
    assert pw[1, 150].sum() < 0.2 and pw[1, 399].sum() < 0.2  # the sink holds head 1
    # sensitivity: a block one longer or one shorter moves the marked rows
    for size in (chunk - 1, chunk + 1):
        off = ob.chunked_sink_attention(w, "m.", dict(mc, mask={"size": size}), h.double().numpy())
        row = 183 if size < chunk else 210  # (key 179 comes into view of 183; key 180 drops out of 210's)
        assert err(off[row], ref[row]) > 0.2
    lim = 3e-2 if dtype == BF16 else 2e-5
    marked = sorted({q for q, _ in inside | outside})
    # (second cut: 178, 183, 358, 361, 398 and 399 are decoded alone, 170 starts a portion)
    for portions in ([400], [170, 8, 1, 4, 1, 156, 18, 1, 2, 1, 36, 1, 1]):
        mixer, cache = _attn_mixer(w, mc, t, device, dtype)
        got = run_mixer(mixer, cache, h, portions, device)
        assert err(got, ref) < lim
        for qi in marked:
            assert err(got[qi], ref[qi]) < lim * 2, (portions[0], qi)


def _mlstm_weights(g, heads, dim, vdim, d, gate_std):
    r = lambda *s, sc: torch.randn(*s, generator=g) * sc  # noqa: E731
    return {"m.q": r(heads * dim, d, sc=0.4), "m.k": r(heads * dim, d, sc=0.4), "m.v": r(heads * vdim, d, sc=0.4),
            "m.g": r(heads * vdim, d, sc=0.4), "m.i": r(heads, d, sc=gate_std), "m.i.b": r(heads, sc=1.0),
            "m.f": r(heads, d, sc=gate_std), "m.f.b": r(heads, sc=1.0) + 2.0,
            "m.norm": torch.rand(heads * vdim, generator=g) + 0.5, "m.o": r(d, heads * vdim, sc=0.2)}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim,vdim,cap,gate_std", [(3, 8, 12, 4.0, 0.3), (1, 40, 8, 15.0, 0.3), (2, 16, 16, 1.5, 1.0),
                                                         (5, 70, 33, 9.0, 2.0), (2, 130, 4, 6.0, 0.5)])
def test_matrix_lstm_mechanism(device, heads, dim, vdim, cap, gate_std):
    """One matrix-memory sublayer against the oracle in portions: key sizes on both sides of the 16-row slices, gates
    inside and far beyond their caps, a running maximum that starts at 0 and is carried across portions."""
    mc = _mls(heads, dim, vdim, cap)
    t, d, eps = 75, 48, 1e-6
    g = torch.Generator().manual_seed(5)
    w = _mlstm_weights(g, heads, dim, vdim, d, gate_std)
    h = torch.randn(t, d, generator=g)
    ref = ob.mlstm(w, "m.", mc, h.double().numpy(), eps)
    if gate_std >= 1.0:
        assert (np.abs(h.double().numpy() @ w["m.i"].double().numpy().T) > cap).any()  # the caps do act
    for portions in ([75], [11, 1, 2, 39, 1, 1, 20], [1] * 75):
        cache = HybridCache([("mlstm", heads, dim, vdim)], 1, t, device, F32)
        mixer = MatrixLSTM(0, heads, dim, vdim, cap, eps,
                           torch.cat([w["m." + n] for n in ("q", "k", "v", "g", "i", "f")]).to(device),
                           torch.cat([w["m.i.b"], w["m.f.b"]]).to(device), w["m.norm"].to(device), w["m.o"].to(device))
        assert err(run_mixer(mixer, cache, h, portions, device), ref) < 2e-5, portions


def _timemix_weights(g, heads, dim, d, rank):
    r = lambda *s, sc: torch.randn(*s, generator=g) * sc  # noqa: E731
    hd = heads * dim
    w = {"m." + n: r(hd, d, sc=0.4) for n in ("r", "k", "v", "g")}
    w.update({"m.mu." + n: torch.rand(d, generator=g) for n in ("r", "k", "v", "g", "w")})
    w.update({"m.w1": r(rank, d, sc=0.4), "m.w2": r(hd, rank, sc=1.0), "m.w0": torch.rand(hd, generator=g) * 5.0 - 4.5,
              "m.u": r(heads, dim, sc=0.5), "m.norm": torch.rand(hd, generator=g) + 0.5, "m.o": r(d, hd, sc=0.2)})
    return w


def _timemix_mixer(w, heads, dim, d, eps, device, dtype=F32):
    mu = torch.stack([w["m.mu." + n] for n in ("r", "k", "v", "g", "w")]).to(device)
    return TimeMix(0, heads, dim, eps, mu, torch.stack([w["m." + n] for n in ("r", "k", "v", "g")]).to(device, dtype),
                   w["m.w1"].to(device, dtype), w["m.w2"].to(device, dtype), w["m.w0"].reshape(heads, dim).to(device),
                   w["m.u"].to(device), w["m.norm"].to(device), w["m.o"].to(device, dtype))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim,rank", [(3, 8, 5), (2, 16, 1), (1, 64, 16), (2, 40, 7), (17, 24, 3), (1, 136, 4)])
def test_time_mix_mechanism(device, heads, dim, rank):
    """One time-mix sublayer against the oracle in portions: the previous token's input carried across portions (zeros
    before the first token), decays from nearly 0 to nearly 1, the bonus for the current token."""
    t, d, eps = 75, 48, 1e-6
    g = torch.Generator().manual_seed(6)
    w = _timemix_weights(g, heads, dim, d, rank)
    h = torch.randn(t, d, generator=g)
    ref = ob.time_mix(w, "m.", {"heads": heads, "dim": dim}, h.double().numpy(), eps)
    for portions in ([75], [11, 1, 2, 39, 1, 1, 20], [1] * 75, [2] * 37 + [1]):
        cache = HybridCache([("timemix", heads, dim, dim, d)], 1, t, device, F32)
        mixer = _timemix_mixer(w, heads, dim, d, eps, device)
        assert err(run_mixer(mixer, cache, h, portions, device), ref) < 2e-5, portions


@pytest.mark.gpu
@pytest.mark.parametrize("seg_min", [4, 8, 16])
def test_scans_cut_into_segments(seg_min, monkeypatch):
    """Both recurrences with a prompt's tokens dealt to segments that run side by side (each segment's own final state
    and decay product, their combination from the carried state, then the scan proper): many short segments, an uneven
    last one, a second portion that starts from a carried state, against the oracle."""
    monkeypatch.setattr(hy, "SCAN_SEG_MIN", seg_min)
    t, d, eps, device = 75, 48, 1e-6, "cuda"
    g = torch.Generator().manual_seed(11)
    h = torch.randn(t, d, generator=g)
    for heads, dim, vdim, cap in [(3, 8, 12, 4.0), (2, 40, 33, 9.0), (1, 130, 4, 2.0)]:
        w = _mlstm_weights(g, heads, dim, vdim, d, 1.0)
        ref = ob.mlstm(w, "m.", _mls(heads, dim, vdim, cap), h.double().numpy(), eps)
        for portions in ([75], [40, 35], [9, 66]):
            assert hy._scan_segments(1, portions[-1], heads, dim, vdim + 1, device)[0] > 1
            cache = HybridCache([("mlstm", heads, dim, vdim)], 1, t, device, F32)
            mixer = MatrixLSTM(0, heads, dim, vdim, cap, eps,
                               torch.cat([w["m." + n] for n in ("q", "k", "v", "g", "i", "f")]).to(device),
                               torch.cat([w["m.i.b"], w["m.f.b"]]).to(device), w["m.norm"].to(device), w["m.o"].to(device))
            assert err(run_mixer(mixer, cache, h, portions, device), ref) < 2e-5, (heads, dim, portions)
    for heads, dim, rank in [(3, 8, 5), (2, 40, 7), (1, 136, 4)]:
        w = _timemix_weights(g, heads, dim, d, rank)
        ref = ob.time_mix(w, "m.", {"heads": heads, "dim": dim}, h.double().numpy(), eps)
        for portions in ([75], [40, 35], [9, 66]):
            cache = HybridCache([("timemix", heads, dim, dim, d)], 1, t, device, F32)
            assert err(run_mixer(_timemix_mixer(w, heads, dim, d, eps, device), cache, h, portions, device), ref) < 2e-5, \
                (heads, dim, portions)


@pytest.mark.parametrize("device", DEVICES)
def test_side_by_side_mixers_share_one_projection(device):
    """Attention and time mix on one input, summed with unequal weights through one output projection."""
    t, d, eps = 30, 48, 1e-6
    left = _left(4, 2, 12, 8, 6, 7)
    mc = _par(left, 3, 8, 0.6, 1.7)
    g = torch.Generator().manual_seed(8)
    wl, wr = _attn_weights(g, left, d), _timemix_weights(g, 3, 8, d, 4)
    w = {k.replace("m.", "x.left."): v for k, v in wl.items()}
    w.update({k.replace("m.", "x.right.", 1): v for k, v in wr.items()})
    h = torch.randn(t, d, generator=g)
    ref = ob.parallel_mixer(w, "x.", mc, h.double().numpy(), eps)
    cache = HybridCache([("multi", ("kv", 2, 12, 8), ("timemix", 3, 8, 8, d))], 1, t, device, F32)
    a, _ = _attn_mixer(wl, left, t, device)
    both = SideBySide([a, _timemix_mixer(wr, 3, 8, d, eps, device)], [0.6, 1.7])
    assert both.w_o.shape == (d, 4 * 8 + 3 * 8)
    assert err(run_mixer(both, cache, h, [13, 1, 2, 14], device), ref) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("m", [1, 5, 70, 300])
def test_clamped_feed_forward(device, m):
    d, ff, limit = 40, 56, 0.9
    g = torch.Generator().manual_seed(4)
    w = {"f.gate": torch.randn(ff, d, generator=g) * 0.5, "f.up": torch.randn(ff, d, generator=g) * 0.5,
         "f.down": torch.randn(d, ff, generator=g) * 0.3}
    x = torch.randn(m, d, generator=g)
    pre = x.double().numpy() @ w["f.up"].double().numpy().T
    assert (pre > limit).any() and (pre < -limit).any()  # the clamps do act
    ref = ob.feed_forward(w, "f.", {"limit": limit}, x.double().numpy())
    blk = GatedDenseFF(torch.cat([w["f.gate"], w["f.up"]]).to(device), w["f.down"].to(device), limit, GATE_ALPHA)
    assert err(blk(x.to(device), None).cpu().numpy(), ref) < 2e-5
    res = x.clone().to(device)  # the residual add in the projection's epilogue
    hy.linear_add_(res, blk.features(x.to(device), None), blk.w_o)
    assert err(res.cpu().numpy(), x.double().numpy() + ref) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
def test_soft_capped_linear(device):
    g = torch.Generator().manual_seed(2)
    x, w = torch.randn(9, 40, generator=g) * 3.0, torch.randn(24, 40, generator=g)
    ref = 2.5 * np.tanh(x.double().numpy() @ w.double().numpy().T / 2.5)
    assert err(hy.linear(x.to(device), w.to(device), act=hy.ACT_SOFTCAP, limit=2.5).cpu().numpy(), ref) < 2e-5
    assert err(hy.linear_softcap(x.to(device), w.to(device), 2.5).cpu().numpy(), ref) < 2e-5
    y = (x @ w.t()).to(device).contiguous()
    assert err(hy.softcap_(y, 2.5).cpu().numpy(), ref) < 2e-5


# ---------------------------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare, cfg_odd])
def test_prompt_logits_and_residual_stream(device, cfg):
    model, sd = build(cfg(), device)
    t = toks(45, model.config.vocab_size)
    ref, ref_hidden = ob.forward(cfg(), sd, t)
    out = model(torch.tensor([t], dtype=torch.int32), output_hidden_states=True)
    for i, hs in enumerate(out.hidden_states):
        assert err(hs[0].cpu().numpy(), ref_hidden[i]) < tol(device), f"layer {i}"
    assert err(out.logits[0].cpu().numpy(), ref) < tol(device)
    assert err(out.logits[0, :3].cpu().numpy(), ref[:3]) < tol(device)  # the first tokens of a sequence
    assert np.abs(ref).max() > 0.8 * cfg()["logit_softcap"] or cfg is not cfg_full  # the cap does act


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_serving_format(device):
    model, sd = build(cfg_full(), device, dtype=BF16)
    t = toks(40, 61)
    ref, _ = ob.forward(cfg_full(), sd, t)
    assert err(run_portions(model, t, [33] + [1] * 7), ref) < tol(device, BF16)
    cache = model.init_cache(1, 8)
    k, v = cache.layer(0)
    assert k.dtype == BF16 and k.shape == (1, 2, 8, 12) and v.shape == (1, 2, 8, 8)
    state, prev = cache.recurrent(0)
    assert state.dtype == F32 and state.shape == (1, 3, 8, 8) and prev.shape == (1, 48)
    state, mrun = cache.recurrent(1)
    assert state.dtype == F32 and state.shape == (1, 3, 8, 13) and mrun.shape == (1, 3)
    assert cache.nbytes() == model.cache_nbytes(1, 8)
    lw = model.blocks[0].mixer.members
    assert lw[0].sink.dtype == F32 and lw[0].temp.dtype == F32 and lw[1].w0.dtype == F32 and lw[1].mu.dtype == F32
    assert model.blocks[1].mixer.gate_bias.dtype == F32 and model.blocks[1].mixer.w_in.dtype == BF16


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare, cfg_odd])
def test_prefill_against_token_by_token(device, cfg):
    model, sd = build(cfg(), device)
    t = toks(34, model.config.vocab_size, seed=2)
    ref, _ = ob.forward(cfg(), sd, t)
    whole = run_portions(model, t, [34])
    single = run_portions(model, t, [1] * 34)
    assert err(whole, ref) < tol(device) and err(single, ref) < tol(device)
    assert err(single, whole) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("portions", [[2] * 20, [3, 2, 9, 1, 1, 17, 2, 5], [12, 13, 14, 1], [1, 39], [38, 2], [7, 7, 7, 7, 7, 5]])
def test_portions_of_any_size(device, portions):
    model, sd = build(cfg_full(), device, seed=1)
    t = toks(sum(portions), 61, seed=3)
    ref, _ = ob.forward(cfg_full(), sd, t)
    assert err(run_portions(model, t, portions), ref) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(device):
    """150 single-token steps after a short prompt: across many block edges of both attention layers (7 and 16), past
    the 64-key runs of the decode kernels, a recurrent state carried 150 times."""
    model, sd = build(cfg_full(), device, seed=2)
    t = toks(156, 61, seed=4)
    ref, _ = ob.forward(cfg_full(), sd, t)
    got = run_portions(model, t, [6] + [1] * 150)
    e = [err(got[i], ref[i]) for i in range(156)]
    assert max(e) < tol(device), int(np.argmax(e))


@pytest.mark.parametrize("device", DEVICES)
def test_rows_are_reset_and_reused(device):
    """A finished request's cache row (keys, values, both kinds of recurrent state, the running maximum, the previous
    token's input) serves the next request from a clean start; two live requests fed in turns do not touch each other."""
    model, sd = build(cfg_full(), device)
    a, b = toks(21, 61, seed=6), toks(17, 61, seed=7)
    ref_a, _ = ob.forward(cfg_full(), sd, a)
    ref_b, _ = ob.forward(cfg_full(), sd, b)
    st = SequenceStepper(model, 32)
    assert err(run_portions(model, a, [20, 1], "a", st), ref_a) < tol(device)
    assert st.live() == [] and len(st._free) == 1
    assert err(run_portions(model, b, [5, 12], "b", st), ref_b) < tol(device)  # the same row again, shorter
    assert len(st._free) == 1
    got_a, got_b = [], []
    for lo in range(0, 21, 3):  # interleaved: two rows live at once, requests of unequal length
        got_a.append(st.feed("a", a[lo:lo + 3], list(range(len(a[lo:lo + 3])))).cpu())
        if lo < 17:
            got_b.append(st.feed("b", b[lo:lo + 3], list(range(len(b[lo:lo + 3])))).cpu())
    assert st.live() == ["a", "b"] and st.held("a") == 21 and st.held("b") == 17
    assert err(torch.cat(got_a).numpy(), ref_a) < tol(device) and err(torch.cat(got_b).numpy(), ref_b) < tol(device)
    with pytest.raises(ValueError):
        st.feed("a", toks(12, 61), [])  # more than the row holds


@pytest.mark.parametrize("device", DEVICES)
def test_batch_rows_against_each_alone(device):
    model, sd = build(cfg_full(), device)
    rows = [toks(19, 61, seed=8), toks(19, 61, seed=9), toks(19, 61, seed=10)]
    cache = model.init_cache(3, 24)
    out = model(torch.tensor(rows, dtype=torch.int32), past_key_values=cache).logits
    nxt = [[5], [6], [7]]
    out2 = model(torch.tensor(nxt, dtype=torch.int32), past_key_values=cache).logits  # one decode step of the batch
    for r in range(3):
        ref, _ = ob.forward(cfg_full(), sd, rows[r] + nxt[r])
        assert err(out[r].cpu().numpy(), ref[:19]) < tol(device)
        assert err(out2[r].cpu().numpy(), ref[19:]) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare])
def test_greedy_generation_through_the_engine(device, cfg):
    """model.generate (prefill + decode steps of the engine, hipGraph replay on the GPU): every generated token is the
    oracle's argmax of the sequence so far (up to rounding between near-equal logits)."""
    model, sd = build(cfg(), device)
    v = model.config.vocab_size
    prompt = toks(9, v, seed=11)
    seq = model.generate(torch.tensor([prompt], dtype=torch.int32),
                         generation_config=GenerationConfig(max_length=30, pad_token_id=0)).sequences[0].cpu().tolist()
    assert seq[:9] == prompt and len(seq) == 30 and all(0 <= x < v for x in seq)
    ref, _ = ob.forward(cfg(), sd, seq)
    for i in range(9, 30):
        row = ref[i - 1]
        assert row.max() - row[seq[i]] <= 1e-4 * np.abs(row).max(), i
    again = model.generate(torch.tensor([prompt], dtype=torch.int32),
                           generation_config=GenerationConfig(max_length=30, pad_token_id=0)).sequences[0].cpu().tolist()
    assert again == seq  # the engine's cached cache row starts clean


@pytest.mark.parametrize("device", DEVICES)
def test_sampled_generation_through_the_engine(device):
    model, sd = build(cfg_full(), device)
    prompt = torch.tensor([toks(7, 61, seed=14)], dtype=torch.int32)
    gc = dict(max_length=27, pad_token_id=0, do_sample=True, temperature=0.9, top_k=5, top_p=0.95)
    a = model.generate(prompt, generation_config=GenerationConfig(seed=3, **gc)).sequences[0].cpu().tolist()
    b = model.generate(prompt, generation_config=GenerationConfig(seed=3, **gc)).sequences[0].cpu().tolist()
    c = model.generate(prompt, generation_config=GenerationConfig(seed=4, **gc)).sequences[0].cpu().tolist()
    assert a == b and a != c and all(0 <= x < 61 for x in a + c)
    ref, _ = ob.forward(cfg_full(), sd, a)
    for i in range(7, 27):
        row = ref[i - 1]
        assert row[a[i]] >= np.sort(row)[-5] - 1e-4 * np.abs(row).max(), i


def test_checkpoint_directory_round_trip(tmp_path):
    from jax_llama_amd.models import registry
    model, sd = build(cfg_full(), "cpu")
    model.save_pretrained(str(tmp_path), sd)
    assert registry.architecture_of(str(tmp_path)) == "besulix"
    again = registry.load_model(str(tmp_path), device="cpu", dtype=F32)
    ids = torch.tensor([toks(12, 61)], dtype=torch.int32)
    assert torch.equal(again(ids).logits, model(ids).logits)
    assert registry.supports_dtype("besulix", F32) and registry.supports_dtype("besulix", BF16)
    assert again.weight_bytes() == model.weight_bytes() > 0
    sd2 = dict(sd)
    sd2["l1.mix.q"] = sd["l1.mix.q"][:-1]
    with pytest.raises(ValueError):
        BesulixForCausalLM(model.config, _do_init=False).load_state_dict(sd2)


def test_trace_runner_program(tmp_path):
    """bin/trace_run as a user starts it: steps on standard input, logits files, 'done' lines, rows given back."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    model, sd = build(cfg_full(), "cpu")
    ckpt, out = str(tmp_path / "ckpt"), str(tmp_path / "out")
    model.save_pretrained(ckpt, sd)
    a, b = toks(19, 61, seed=12), toks(5, 61, seed=13)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [0, 10]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b, "want": [4]}], "end": ["b"]}]
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", ckpt, "--dtype", "float32",
                        "--out", out, "--max-tokens", "24", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not os.path.exists(os.path.join(out, "1.f32"))
    ref_a, _ = ob.forward(cfg_full(), sd, a)
    ref_b, _ = ob.forward(cfg_full(), sd, b)
    got0 = np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, 61)
    got2 = np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(2, 61)
    got3 = np.fromfile(os.path.join(out, "3.f32"), dtype="<f4").reshape(1, 61)
    assert err(got0, ref_a[[0, 5]]) < 2e-5 and err(got2, ref_a[[8, 18]]) < 2e-5 and err(got3, ref_b[[4]]) < 2e-5


def cfg_kernel_shapes():
    """Head sizes of the MFMA attention kernels beside ones of the plain kernels, blocks that end inside tiles, key
    sizes of the scans from one 16-row slice to eight, six layers in another order."""
    return {"architecture": "Besulix", "vocab": 300, "width": 192, "norm": {"eps": 1e-6}, "logit_softcap": 12.0,
            "layers": [{"type": "mlstm", "mixer": _mls(4, 32, 48, 8.0), "mlp": _ff(320, 1.5)},
                       {"type": "parallel", "mixer": _par(_left(6, 2, 64, 64, 32, 150, 0.12, 1e4), 3, 64, 0.8, 0.5), "mlp": None},
                       {"type": "parallel", "mixer": _par(_left(4, 4, 48, 80, 48, 37, 0.15, 500.0), 6, 32, 1.2, 0.9),
                        "mlp": _ff(100, 4.0)},
                       {"type": "mlstm", "mixer": _mls(2, 128, 64, 12.0), "mlp": None},
                       {"type": "parallel", "mixer": _par(_left(2, 1, 128, 128, 64, 256, 0.09, 1e6), 1, 128, 0.5, 1.0),
                        "mlp": _ff(64, 2.0)},
                       {"type": "mlstm", "mixer": _mls(6, 16, 32, 3.0), "mlp": _ff(192, 0.7)}]}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_longer_prompts_at_the_kernel_shapes(dtype):
    """600 tokens in uneven portions (prompt-sized GEMMs, the flash prefill starting at unaligned slots and crossing
    block edges inside a wave's queries, decode over several key runs) on the GPU against the framework's fp32 CPU path,
    which the tests above tie to the oracle."""
    cfg = cfg_kernel_shapes()
    ref_model, sd = build(cfg, "cpu", F32, decay_rank=32)  # (a rank the packed GEMM takes: its soft cap is a pass of its own)
    t = toks(600, 300, seed=21)
    with torch.no_grad():
        ref = ref_model(torch.tensor([t], dtype=torch.int32)).logits[0].numpy()
    model = BesulixForCausalLM(BesulixConfig.from_dict(cfg), device="cuda", dtype=dtype, _do_init=False).load_state_dict(sd)
    got = run_portions(model, t, [261, 3, 2, 190, 64, 37] + [1] * 43)
    e = np.array([err(got[i], ref[i]) for i in range(600)])
    # (bf16: six layers of rounded operands; the largest of 600 rows sits a few times above the typical one, while a
    # wrong mask, state or position puts a row at order 1)
    assert e.max() < (2e-4 if dtype == F32 else 8e-2), (int(np.argmax(e)), e.max())
    assert e.mean() < (5e-5 if dtype == F32 else 1.5e-2), e.mean()
    whole = run_portions(model, t, [600])
    assert err(whole, got) < (2e-5 if dtype == F32 else 2e-2)
