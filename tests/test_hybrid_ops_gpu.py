"""The hybrid-mixer HIP kernels (jax_llama_amd._C_hybrid) against the PyTorch implementation of the same ops
(ops/hybrid.py CPU path), at sizes that are not multiples of the tile shapes, in both number formats."""
import pytest
import torch

from jax_llama_amd.ops import hybrid as hy

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dt):
    return 2e-5  # both paths round the operands alike: only the summation order differs


def _close(a, b, tol, what=""):
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape, f"{what}: shapes {tuple(a.shape)} vs {tuple(b.shape)}"
    if a.numel() == 0:
        return
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-6))
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


def _rand(*shape, dt=torch.float32, std=1.0):
    return (torch.randn(*shape) * std).to(dt)


def test_extension_loaded():
    assert hy.ext_available() and hy.so_path().endswith(".so")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 7, 24), (3, 64, 320), (8, 130, 72), (9, 4, 320), (70, 392, 320), (200, 96, 24),
                                   (129, 64, 257), (600, 200, 96), (513, 130, 320)])
def test_linear(dt, m, n, k):
    x, w = _rand(m, k), _rand(n, k, dt=dt, std=k ** -0.5)
    _close(hy.linear(x.to(DEV), w.to(DEV)), hy.linear(x, w), _tol(dt), "linear")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m", [2, 8, 77, 530])
def test_linear_swiglu_strided_rows(dt, m):
    k, n = 96, 40
    big = _rand(m, k + 32)
    w = _rand(2 * n, k, dt=dt, std=k ** -0.5)
    got = hy.linear(big.to(DEV)[:, 16:16 + k], w.to(DEV), swiglu=True)
    _close(got, hy.linear(big[:, 16:16 + k], w, swiglu=True), _tol(dt), "swiglu")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,top,e", [(1, 2, 8), (4, 2, 8), (3, 1, 1), (150, 2, 8), (90, 3, 5), (300, 1, 4),
                                     (20, 2, 8), (21, 3, 2), (9, 1, 1), (700, 2, 3)])
def test_moe_table(dt, m, top, e):
    d, ff, v = 72, 40, 50
    x = _rand(m, d)
    ids = torch.randint(0, v, (m,), dtype=torch.int32)
    table = torch.stack([torch.randperm(e)[:top] for _ in range(v)]).to(torch.int32)
    w_gu, w_down = _rand(e, 2 * ff, d, dt=dt, std=d ** -0.5), _rand(e, d, ff, dt=dt, std=ff ** -0.5)
    got = hy.moe_table(x.to(DEV), ids.to(DEV), table.to(DEV), w_gu.to(DEV), w_down.to(DEV))
    # bf16: the hidden activation is rounded to bf16 before the down projection on both paths, but the two paths'
    # fp32 sums differ in order, so a hidden value can round to the neighbouring bf16
    _close(got, hy.moe_table(x, ids, table, w_gu, w_down), 2e-5 if dt == torch.float32 else 4e-3, "moe")


@pytest.mark.parametrize("wn", [1, 50])
@pytest.mark.parametrize("nsum", [1, 3])
def test_norm_residual(wn, nsum):
    m, d = 5, 50
    x, y, w = _rand(m, d), _rand(m * nsum, d), torch.rand(wn) + 0.5
    got = hy.norm_residual_(x.clone().to(DEV), y.to(DEV), w.to(DEV), 1e-6, nsum, 1.0 / nsum)
    _close(got, hy.norm_residual_(x.clone(), y, w, 1e-6, nsum, 1.0 / nsum), 1e-5, "norm_residual")
    _close(hy.rms_rows(y.to(DEV), w.to(DEV), 1e-6), hy.rms_rows(y, w, 1e-6), 1e-5, "rms_rows")


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_and_side_gate(dt):
    v, d, m = 40, 30, 6
    table = _rand(v, 3 * d, dt=dt)
    ids = torch.randint(0, v, (m,), dtype=torch.int32)
    _close(hy.embed_rows(ids.to(DEV), table.to(DEV), d, d), hy.embed_rows(ids, table, d, d), 0.0, "embed")
    gp = _rand(m, d)
    _close(hy.gelu_gate_rows(gp.to(DEV), ids.to(DEV), table.to(DEV), 2 * d), hy.gelu_gate_rows(gp, ids, table, 2 * d),
           1e-5, "gelu gate")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [dict(b=1, s=1, s0=0, h=4, g=2, dim=64, vdim=64),
                                   dict(b=2, s=5, s0=0, h=3, g=1, dim=24, vdim=40),
                                   dict(b=1, s=70, s0=130, h=4, g=4, dim=72, vdim=136),
                                   dict(b=2, s=1, s0=300, h=6, g=2, dim=32, vdim=16),
                                   dict(b=1, s=70, s0=130, h=4, g=2, dim=64, vdim=128),   # the MFMA prefill shapes
                                   dict(b=2, s=203, s0=0, h=2, g=1, dim=128, vdim=64),
                                   dict(b=1, s=33, s0=31, h=2, g=2, dim=128, vdim=128)])
@pytest.mark.parametrize("own_kv", [True, False])
def test_attention(dt, shape, own_kv):
    b, s, s0, h, g, dim, vdim = (shape[k] for k in ("b", "s", "s0", "h", "g", "dim", "vdim"))
    t, eps = s0 + s + 3, 1e-6
    kc, vc = _rand(b, g, t, dim, dt=dt), _rand(b, g, t, vdim, dt=dt)
    cols = h * dim + (g * (dim + vdim) if own_kv else 0)
    proj = _rand(b * s, cols)
    pos = (torch.arange(s0, s0 + s, dtype=torch.int32)[None] + torch.zeros(b, 1, dtype=torch.int32)).contiguous()
    bias = hy.distance_bias_table(_rand(10, h), 37)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    q_ref = hy.attn_prep(proj, pos, s0, b, s, h, g, dim, vdim, kc if own_kv else None, vc if own_kv else None, eps,
                         0.3, 4)
    q_got = hy.attn_prep(proj.to(DEV), pos.to(DEV), s0, b, s, h, g, dim, vdim, kc_g if own_kv else None,
                         vc_g if own_kv else None, eps, 0.3, 4)
    _close(q_got, q_ref, 1e-5, "q")
    _close(kc_g, kc, 1e-5 if dt == torch.float32 else 8e-3, "k cache")
    _close(vc_g, vc, 1e-5 if dt == torch.float32 else 8e-3, "v cache")
    # the attention itself on identical caches
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    # bf16 caches at the MFMA shapes: q is rounded to bf16 for the score product (the reference gets the same q)
    mma = dt == torch.bfloat16 and s > 1 and dim in (64, 128) and vdim in (64, 128)
    for cap, b_ in ((5.0, bias), (0.0, None)):
        ref = hy.attn_bias(q_ref.to(torch.bfloat16).float() if mma else q_ref, kc, vc, s0, 0.25, cap, b_)
        got = hy.attn_bias(q_ref.to(DEV), kc_g, vc_g, torch.tensor([s0], dtype=torch.int32, device=DEV), 0.25, cap,
                           b_.to(DEV) if b_ is not None else None)
        _close(got, ref, 2e-4 if mma else 2e-5, "attention")  # (MFMA path: v_exp_f32 and exp-based tanh)


@pytest.mark.parametrize("shape", [dict(b=1, s=1, h=4, g=2, dim=32, vdim=32, taps=4),
                                   dict(b=2, s=2, h=2, g=1, dim=40, vdim=24, taps=4),
                                   dict(b=1, s=37, h=6, g=3, dim=128, vdim=72, taps=3),
                                   dict(b=2, s=9, h=2, g=2, dim=16, vdim=130, taps=1)])
def test_delta_rule(shape):
    b, s, h, g, dim, vdim, taps = (shape[k] for k in ("b", "s", "h", "g", "dim", "vdim", "taps"))
    c = 2 * g * dim + h * vdim
    proj = _rand(b * s, c + h * vdim + 2 * h + 5)[:, :c + h * vdim + 2 * h]  # strided rows
    conv_w, tail = _rand(c, taps, std=0.6), _rand(b, c, max(taps - 1, 0))
    a_log, dt_bias = torch.rand(h) - 1.0, torch.randn(h)
    state = _rand(b, h, dim, vdim, std=0.3)
    tail_g, state_g = tail.clone().to(DEV), state.clone().to(DEV)
    ref = hy.delta_prep(proj, b, s, h, g, dim, vdim, conv_w, tail, a_log, dt_bias)
    got = hy.delta_prep(proj.to(DEV), b, s, h, g, dim, vdim, conv_w.to(DEV), tail_g, a_log.to(DEV), dt_bias.to(DEV))
    for r, x, name in zip(ref, got, ("q", "k", "v", "beta", "decay")):
        _close(x, r, 2e-5, name)
    _close(tail_g, tail, 0.0, "conv tail")
    o_ref = hy.delta_scan(*ref, state, b, s)
    o_got = hy.delta_scan(*(x.to(DEV) for x in ref), state_g, b, s)
    _close(o_got, o_ref, 5e-5, "delta o")
    _close(state_g, state, 5e-5, "delta state")
    gate, w = _rand(b * s, h * vdim), torch.rand(vdim) + 0.5
    _close(hy.gated_rmsnorm(o_ref.to(DEV), gate.to(DEV), w.to(DEV), 1e-6), hy.gated_rmsnorm(o_ref, gate, w, 1e-6), 2e-5,
           "gated norm")


@pytest.mark.parametrize("m,n,k", [(256, 64, 96), (777, 400, 320), (2048, 16, 32)])
def test_linear_on_the_packed_gemm(m, n, k):
    """Prompt-sized dense bf16 linears go to the framework's fragment-packed MFMA GEMM when the main extension is
    built; same operands, so the result matches the row-major kernel and the CPU op up to summation order."""
    from jax_llama_amd import ops
    x, w = _rand(m, k), _rand(n, k, dt=torch.bfloat16, std=k ** -0.5)
    xg, wg = x.to(DEV), w.to(DEV)
    assert hy._use_packed_gemm(xg, wg) == ops.ext_available()
    got = hy.linear(xg, wg)
    _close(got, hy.linear(x, w), 2e-5, "packed gemm vs cpu")
    hy.PACKED_GEMM = False
    try:
        _close(hy.linear(xg, wg), got, 2e-5, "row-major kernel vs packed gemm")
    finally:
        hy.PACKED_GEMM = True
    assert not hy._use_packed_gemm(xg[:100], wg) and not hy._use_packed_gemm(xg, wg[:15])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m", [1, 8, 77, 530])
@pytest.mark.parametrize("act", [hy.ACT_RELU2, hy.ACT_CLAMP_GLU])
def test_linear_activations(dt, m, act):
    """Squared ReLU (one accumulator) and the clamped gated form (two), pre-activations on both sides of the clamps."""
    k, n = 96, 40
    x = _rand(m, k)
    w = _rand(n * (2 if hy.act_gated(act) else 1), k, dt=dt, std=2.0 * k ** -0.5)
    got = hy.linear(x.to(DEV), w.to(DEV), act=act, limit=1.3, alpha=1.702)
    ref = hy.linear(x, w, act=act, limit=1.3, alpha=1.702)
    assert float(ref.abs().max()) > 0
    _close(got, ref, _tol(dt), "activation")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,h,k,n", [(1, 3, 16, 40), (1, 12, 24, 8), (1, 70, 8, 16), (5, 8, 64, 128), (33, 5, 40, 24),
                                     (300, 6, 128, 48), (9, 70, 8, 16)])
def test_heads_linear(dt, m, h, k, n):
    x, w = _rand(m, h, k), _rand(h, n, k, dt=dt, std=k ** -0.5)
    _close(hy.heads_linear(x.to(DEV), w.to(DEV)), hy.heads_linear(x, w), _tol(dt), "per-head linear")


@pytest.mark.parametrize("m,e,top", [(1, 4, 2), (7, 1, 1), (40, 12, 1), (300, 70, 5), (9, 1024, 8), (65, 5, 5)])
def test_route_topk(m, e, top):
    """The score router's record: chosen experts by descending logit, sigmoid weights, and an expert-sorted order that
    is a permutation of the (token, choice) rows with the right offsets."""
    z = _rand(m, e + 3, std=2.0)[:, :e + 1]  # strided rows, one extra column that is not an expert
    ex_ref, w_ref = hy.route_topk(z, e, top)
    r = m * top
    idx = torch.empty(4 * r + e + 1, dtype=torch.int32, device=DEV)
    wts = torch.empty(2 * r, dtype=torch.float32, device=DEV)
    hy.ext().route_topk(z.to(DEV), e, top, idx[:r], idx[r:2 * r], wts[:r],
                        idx[2 * r:3 * r], idx[3 * r:4 * r], wts[r:], idx[4 * r:])
    idx, wts = idx.cpu(), wts.cpu()
    row_expert, row_tok, sort_tok, sort_dst, offs = idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]
    assert torch.equal(row_expert.long(), ex_ref) and torch.equal(row_tok.long(), torch.arange(m).repeat_interleave(top))
    _close(wts[:r], w_ref, 1e-6, "router weights")
    assert sorted(sort_dst.tolist()) == list(range(r)) and torch.equal(sort_tok, sort_dst // top)
    assert torch.equal(wts[r:], wts[:r][sort_dst.long()])
    counts = torch.bincount(ex_ref, minlength=e)
    assert offs[0] == 0 and torch.equal(offs[1:].long(), counts.cumsum(0))
    assert torch.equal(row_expert[sort_dst.long()], row_expert[sort_dst.long()].sort().values)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,top,e", [(1, 2, 8), (4, 2, 8), (3, 1, 1), (150, 2, 8), (90, 3, 5), (20, 2, 8), (700, 2, 3)])
def test_moe_routed(dt, m, top, e):
    d, ff = 72, 40
    x, z = _rand(m, d), _rand(m, e + 1, std=2.0)
    w_gu, w_down = _rand(e, 2 * ff, d, dt=dt, std=2.0 * d ** -0.5), _rand(e, d, ff, dt=dt, std=ff ** -0.5)
    got = hy.moe_routed(x.to(DEV), z.to(DEV), top, w_gu.to(DEV), w_down.to(DEV), hy.ACT_CLAMP_GLU, 0.9, 1.702)
    ref = hy.moe_routed(x, z, top, w_gu, w_down, hy.ACT_CLAMP_GLU, 0.9, 1.702)
    _close(got, ref, 2e-5 if dt == torch.float32 else 4e-3, "routed moe")  # (bf16: see test_moe_table)


@pytest.mark.parametrize("gate", [True, False])
def test_norm_residual_with_a_gated_summand(gate):
    m, d, nsum = 7, 50, 2
    x, y, w, extra = _rand(m, d), _rand(m * nsum, d), torch.rand(d) + 0.5, _rand(m, d)
    z = _rand(m, 6)
    g_cpu, g_gpu = (z[:, 4:5], z.to(DEV)[:, 4:5]) if gate else (None, None)
    got = hy.norm_residual_(x.clone().to(DEV), y.to(DEV), w.to(DEV), 1e-6, nsum, 1.0, extra.to(DEV), g_gpu)
    _close(got, hy.norm_residual_(x.clone(), y, w, 1e-6, nsum, 1.0, extra, g_cpu), 1e-5, "norm_residual extra")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("b,s,s0,rank,qc", [(1, 1, 0, 40, 48), (2, 5, 3, 128, 0), (1, 70, 130, 56, 96)])
def test_latent_prep_and_scaled_embedding(dt, b, s, s0, rank, qc):
    t = s0 + s + 2
    proj, w = _rand(b * s, qc + rank + 4), torch.rand(rank) + 0.5
    c_ref = torch.zeros(b, 1, t, rank, dtype=dt)
    c_got = c_ref.clone().to(DEV)
    q_ref = hy.latent_prep(proj, qc, w, s0, b, s, c_ref, 1e-5, q_cols=qc)
    q_got = hy.latent_prep(proj.to(DEV), qc, w.to(DEV), s0, b, s, c_got, 1e-5, q_cols=qc)
    _close(c_got, c_ref, 1e-5 if dt == torch.float32 else 8e-3, "latent cache")
    assert (q_ref is None) == (q_got is None) == (qc == 0)
    if qc:
        _close(q_got, q_ref, 0.0, "q copy")
    table = _rand(30, 24, dt=dt)
    ids = torch.randint(0, 30, (6,), dtype=torch.int32)
    _close(hy.embed_rows(ids.to(DEV), table.to(DEV), scale=7.25), hy.embed_rows(ids, table, scale=7.25), 1e-7, "embed")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [dict(b=1, s=1, s0=0, h=4, rank=64), dict(b=2, s=5, s0=0, h=3, rank=40),
                                   dict(b=1, s=70, s0=130, h=4, rank=136), dict(b=2, s=1, s0=300, h=6, rank=128),
                                   dict(b=1, s=1, s0=700, h=2, rank=24), dict(b=1, s=70, s0=130, h=5, rank=64),
                                   dict(b=2, s=1, s0=1500, h=3, rank=512), dict(b=1, s=1, s0=77, h=5, rank=264),
                                   dict(b=3, s=1, s0=0, h=2, rank=136), dict(b=1, s=1, s0=2100, h=16, rank=384),
                                   dict(b=8, s=1, s0=2100, h=16, rank=264), dict(b=4, s=1, s0=1200, h=32, rank=512),
                                   dict(b=2, s=203, s0=0, h=2, rank=128), dict(b=1, s=33, s0=31, h=12, rank=128)])
def test_attention_with_a_sink_over_one_shared_cache(dt, shape):
    """Keys = values = one cache head, a sink per head (one far above the scores, one far below), prompt and decode
    kernels of every latent size class."""
    b, s, s0, h, rank = (shape[k] for k in ("b", "s", "s0", "h", "rank"))
    t = s0 + s + 3
    c = _rand(b, 1, t, rank, dt=dt)
    q = _rand(b, s, h, rank)
    sink = torch.randn(h) * 2.0
    sink[0], sink[-1] = 25.0, -25.0
    cg = c.to(DEV)
    mma = dt == torch.bfloat16 and s > 1 and rank in (64, 128)
    ref = hy.attn_bias(q.to(torch.bfloat16).float() if mma else q, c, c, s0, 0.1, sink=sink)
    got = hy.attn_bias(q.to(DEV), cg, cg, torch.tensor([s0], dtype=torch.int32, device=DEV), 0.1, sink=sink.to(DEV))
    _close(got, ref, 2e-4 if mma else 2e-5, "sink attention")
    plain = hy.attn_bias(q, c, c, s0, 0.1)
    assert float((plain - ref).abs().max()) > 1e-2  # the sink matters


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,n", [(1, 130), (2, 12), (8, 40), (9, 40), (300, 12), (300, 130), (2, 9000)])
def test_linear_norms_its_input(dt, m, n):
    """An ``RmsInput`` through the GEMV (which norms the rows it reads) and through the tiles (which read the normed
    value) gives what the CPU op gives."""
    k = 200
    x, gain, w = _rand(m, k, std=3.0), torch.rand(k) + 0.5, _rand(n, k, dt=dt, std=k ** -0.5)
    ref = hy.linear(hy.RmsInput(x, gain, 1e-5), w, act=hy.ACT_RELU2)
    h = hy.RmsInput(x.to(DEV), gain.to(DEV), 1e-5)
    got = hy.linear(h, w.to(DEV), act=hy.ACT_RELU2)
    assert (h._value is None) == (m <= hy.FUSE_NORM_MAX_ROWS)
    # bf16: the normed operand is rounded to bf16 on both paths, from fp32 values that differ in the last bit
    _close(got, ref, 2e-5 if dt == torch.float32 else 4e-3, "fused input norm")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,top", [(1, 2), (4, 2), (5, 2)])
def test_moe_routed_norms_its_input(dt, m, top):
    d, ff, e = 72, 40, 6
    x, gain, z = _rand(m, d, std=2.0), torch.rand(d) + 0.5, _rand(m, e, std=2.0)
    w_gu, w_down = _rand(e, 2 * ff, d, dt=dt, std=2.0 * d ** -0.5), _rand(e, d, ff, dt=dt, std=ff ** -0.5)
    ref = hy.moe_routed(hy.RmsInput(x, gain, 1e-5), z, top, w_gu, w_down, hy.ACT_CLAMP_GLU, 0.9, 1.702)
    got = hy.moe_routed(hy.RmsInput(x.to(DEV), gain.to(DEV), 1e-5), z.to(DEV), top, w_gu.to(DEV), w_down.to(DEV),
                        hy.ACT_CLAMP_GLU, 0.9, 1.702)
    _close(got, ref, 2e-5 if dt == torch.float32 else 4e-3, "routed moe, fused input norm")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [  # every attention kernel: plain / fast / shared-latent decode, plain / MFMA prefill
    dict(b=2, s=1, s0=300, h=4, g=2, dim=48, vdim=40), dict(b=1, s=1, s0=700, h=4, g=1, dim=64, vdim=128),
    dict(b=2, s=1, s0=333, h=6, g=1, dim=264, vdim=232, shared=True), dict(b=1, s=1, s0=90, h=3, g=1, dim=96, vdim=64, shared=True),
    dict(b=1, s=70, s0=131, h=4, g=2, dim=48, vdim=40), dict(b=2, s=150, s0=77, h=4, g=2, dim=128, vdim=64),
    dict(b=1, s=100, s0=250, h=2, g=1, dim=96, vdim=64, shared=True)])
@pytest.mark.parametrize("window,keep", [(1, 0), (37, 0), (64, 5), (100, 130), (1000, 3)])
def test_attention_windows_gates_and_wide_value_rows(dt, shape, window, keep):
    """Sliding windows with kept first keys, the gate per (token, head) and values that are the leading columns of the
    key rows (one shared cache), in every attention kernel against the CPU op."""
    b, s, s0, h, g, dim, vdim = (shape[k] for k in ("b", "s", "s0", "h", "g", "dim", "vdim"))
    t = s0 + s + 3
    q = _rand(b, s, h, dim, std=0.5)
    kc = _rand(b, g, t, dim, dt=dt)
    vc = kc if shape.get("shared") else _rand(b, g, t, vdim, dt=dt)
    gate = _rand(b * s, h + 2)[:, 1:h + 1]  # a column view of a wider projection
    kw = dict(window=window, keep_first=keep, vdim=vdim if shape.get("shared") else None)
    kg = kc.to(DEV)
    vg = kg if shape.get("shared") else vc.to(DEV)
    gg = gate.to(DEV)
    for gt, gr in ((gg, gate), (None, None)):
        ref = hy.attn_bias(q, kc, vc, s0, dim ** -0.5, gate=gr, **kw)
        got = hy.attn_bias(q.to(DEV), kg, vg, s0, dim ** -0.5, gate=gt, **kw)
        # (the MFMA prefill rounds q to bf16 for the score product like any other matrix operand)
        mma = dt == torch.bfloat16 and s > 1 and dim in (64, 128) and vdim in (64, 128) and not shape.get("shared")
        _close(got, ref, 2e-2 if mma else 2e-5, f"window {window} keep {keep}")
    with pytest.raises(ValueError):
        hy.attn_bias(q, kc, vc, s0, 1.0, chunk=8, window=4)


@pytest.mark.parametrize("m,e,top,groups,keep", [(1, 10, 2, 5, 3), (7, 1, 1, 1, 1), (40, 12, 4, 4, 2), (300, 64, 5, 8, 3),
                                                 (9, 70, 6, 7, 1), (65, 1000, 8, 10, 4), (33, 20, 4, 4, 3)])
@pytest.mark.parametrize("biased", [True, False])
def test_route_grouped(m, e, top, groups, keep, biased):
    """The grouped softmax router's record (one-pass form up to 64 experts, round-based beyond): the chosen set and the
    weights of the CPU op, and an expert-sorted order that is a permutation of the rows with the right offsets."""
    top = min(top, keep * (e // groups))
    z = _rand(m, e + 3, std=2.0)[:, :e]
    corr = _rand(e, std=0.05) if biased else None
    ex_ref, w_ref = hy.route_grouped(z, corr, top, groups, keep)
    r = m * top
    idx = torch.empty(4 * r + e + 1, dtype=torch.int32, device=DEV)
    wts = torch.empty(2 * r, dtype=torch.float32, device=DEV)
    hy.ext().route_grouped(z.to(DEV), corr.to(DEV) if biased else None, e, top, groups, keep, idx[:r], idx[r:2 * r], wts[:r],
                           idx[2 * r:3 * r], idx[3 * r:4 * r], wts[r:], idx[4 * r:])
    ex, tok, stok, sdst, offs = (x.cpu() for x in (idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]))
    order = torch.argsort(ex.reshape(m, top), 1)
    assert torch.equal(torch.gather(ex.reshape(m, top), 1, order).long(), torch.sort(ex_ref.reshape(m, top), 1).values)
    by_expert = torch.gather(w_ref.reshape(m, top), 1, torch.argsort(ex_ref.reshape(m, top), 1))
    _close(torch.gather(wts[:r].cpu().reshape(m, top), 1, order), by_expert, 1e-5, "weights")
    assert torch.equal(tok, torch.arange(m, dtype=torch.int32).repeat_interleave(top))
    assert int(offs[0]) == 0 and int(offs[e]) == r and torch.equal(torch.sort(sdst).values.long(), torch.arange(r))
    assert torch.equal(ex[sdst.long()], torch.sort(ex).values) and torch.equal(stok, tok[sdst.long()])
    _close(wts[r:], wts[:r][sdst.long().to(DEV)], 0.0, "sorted weights")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,experts,identity,top", [(1, 4, 2, 3), (2, 6, 2, 4), (20, 3, 5, 2), (150, 8, 2, 2), (700, 2, 1, 1)])
def test_moe_grouped_and_the_stream_update(dt, m, experts, identity, top):
    """Experts with identity experts behind them on all three linear paths, summed by the stream update, against the CPU
    ops; the feed-forward of a prompt on the packed GEMM against the row linear."""
    d, ff, streams = 64, 96, 3
    x = _rand(m, d)
    z = _rand(m, experts + identity, std=2.0)
    w_up, w_down = _rand(experts, ff, d, dt=dt, std=d ** -0.5), _rand(experts, d, ff, dt=dt, std=ff ** -0.5)
    y, ex, wt = hy.moe_grouped(x, z, None, top, 1, 1, w_up, w_down)
    yg, exg, wtg = hy.moe_grouped(x.to(DEV), z.to(DEV), None, top, 1, 1, w_up.to(DEV), w_down.to(DEV))
    xs = _rand(streams, m, d)
    mix, ow, nxt, extra = _rand(streams, streams), _rand(streams), _rand(streams), _rand(m, d)
    xg = xs.to(DEV).clone()
    u = hy.hc_update_(xs, mix, ow, y, top, wt, ex, experts, x, extra, next_in=nxt)
    ug = hy.hc_update_(xg, mix.to(DEV), ow.to(DEV), yg, top, wtg, exg, experts, x.to(DEV), extra.to(DEV), next_in=nxt.to(DEV))
    _close(xg, xs, 5e-5, "streams")
    _close(ug, u, 5e-5, "next input")
    s_up, s_down = _rand(ff, d, dt=dt, std=d ** -0.5), _rand(d, ff, dt=dt, std=ff ** -0.5)
    _close(hy.ff_dense(x.to(DEV), s_up.to(DEV), s_down.to(DEV)), hy.ff_dense(x, s_up, s_down), 2e-5, "one-accumulator FF")
