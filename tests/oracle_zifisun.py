"""Plain, slow float64 implementation of the Zifisun decoder for the tests: one function per mechanism, written from
the equations, no cache (a whole sequence is recomputed from its first token; every head's keys and values are
materialised) and no code shared with the package. Inputs: the config as a plain dict (the config.json layout) and a
checkpoint-named dict of tensors.

Equations (eps = norm.eps, rms(y) = y / sqrt(mean(y^2) + eps), n(y; w) = rms(y) * w):
  streams      X_1 .. X_S = embed[token] (S = streams). Sublayer q of a layer (1: mixer, 2: feed-forward) reads
               u = sum_s a_s X_s (a = hc<q>.in), computes y = sublayer(n(u; norm<q>)), and replaces every stream at
               once: X_t <- sum_s B[s, t] X_s + c_t y (B = hc<q>.mix, c = hc<q>.out). The residual is sum_s X_s.
  order        layers 0 .. start-1 once, then layers start .. stop-1 `times` times in a row (same weights), then the rest
  rotation     pair (2i, 2i+1) of a vector at position p turns by the angle p * base^(-2i / dims), i < dims / 2
  latent attn  cq = n(W_dq h; dq.norm); q = W_uq cq, per head [dim plain | rot_dim rotated]
               W_dkv h = [c' (kv_rank) | r (rot_dim)];  c = n(c'; dkv.norm);  r rotated, one per token for all heads
               per head: k_j = W_uk c_j, v_j = W_uv c_j;  s_ij = scale * (q_plain_i . k_j + q_rot_i . r_j)
               j visible from i when 0 <= i - j < mask.size;  softmax over the visible j
               o_i = sigmoid(W_g h_i)[head] * sum_j p_ij v_j;  out = W_o concat(o)
  attention    q = W_q h, k = W_k h, v = W_v h; every q / k head RMS-normed over dim with the weights q.norm / k.norm;
               query head a reads key / value head floor(a / (H / G)); s_ij = scale * q_i . k_j (no positions)
               j visible from i when j <= i and (i - j < mask.size or j < mask.keep_first); gate and output as above
  expert       W_down relu(W_up h)^2
  moe          z = W_router h over experts + identity experts; s = softmax(z); choice c = s + correction
               groups of (experts + identity) / groups.count neighbours, a group's score = its largest c; outside the
               groups.keep best groups c = -inf; the `top` largest c are chosen; weight of a chosen one = its s
               out = sum_chosen s_e * (expert_e(h), or h itself for an identity expert) + shared(h)
  logits       head @ n(sum_s X_s; final.norm)
"""
import numpy as np


def _np(t):
    return t.detach().to("cpu").double().numpy() if hasattr(t, "detach") else np.asarray(t, dtype=np.float64)


def rms(y, eps):
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotate_pairs(x, pos, base, dims):
    """``x [t, ..., n]``: the first ``dims`` numbers of the last axis turned, number 2i with number 2i + 1."""
    out = x.copy()
    for i in range(dims // 2):
        ang = np.asarray(pos, dtype=np.float64) * float(base) ** (-2.0 * i / dims)
        c, s = np.cos(ang), np.sin(ang)
        shape = (-1,) + (1,) * (x.ndim - 2)
        c, s = c.reshape(shape), s.reshape(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i, j, mask):
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    if mask is None or mask.get("size") is None:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def _softmax_attend(q, k, v, scale, mask, pos):
    """One head: ``q [t, d]``, ``k [t, d]``, ``v [t, dv]`` -> ``[t, dv]`` and the weights ``[t, t]``."""
    t = q.shape[0]
    o = np.zeros((t, v.shape[1]))
    w = np.zeros((t, t))
    for i in range(t):
        js = [j for j in range(t) if visible(pos[i], pos[j], mask)]
        s = (k[js] @ q[i]) * scale
        e = np.exp(s - s.max())
        p = e / e.sum()
        w[i, js] = p
        o[i] = p @ v[js]
    return o, w


def latent_attention(w, pre, mc, h, eps, pos=None, return_weights=False):
    t = h.shape[0]
    pos = np.arange(t) if pos is None else np.asarray(pos)
    nh, d, dr, dv = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"]
    rank = mc["kv_rank"]
    cq = rms(h @ _np(w[pre + "dq"]).T, eps) * _np(w[pre + "dq.norm"])
    q = (cq @ _np(w[pre + "uq"]).T).reshape(t, nh, d + dr)
    down = h @ _np(w[pre + "dkv"]).T
    c = rms(down[:, :rank], eps) * _np(w[pre + "dkv.norm"])
    rot = mc["rot"]
    r = rotate_pairs(down[:, rank:rank + dr], pos, rot["base"], rot["dims"])
    q_rot = rotate_pairs(q[:, :, d:], pos, rot["base"], rot["dims"])
    k = (c @ _np(w[pre + "uk"]).T).reshape(t, nh, d)
    v = (c @ _np(w[pre + "uv"]).T).reshape(t, nh, dv)
    gate = sigmoid(h @ _np(w[pre + "g"]).T)
    o = np.zeros((t, nh, dv))
    weights = np.zeros((nh, t, t))
    for a in range(nh):
        qa = np.concatenate([q[:, a, :d], q_rot[:, a]], -1)
        ka = np.concatenate([k[:, a], r], -1)
        oa, weights[a] = _softmax_attend(qa, ka, v[:, a], mc["scale"], mc.get("mask"), pos)
        o[:, a] = oa * gate[:, a:a + 1]
    out = o.reshape(t, nh * dv) @ _np(w[pre + "o"]).T
    return (out, weights) if return_weights else out


def attention(w, pre, mc, h, eps, pos=None, return_weights=False):
    t = h.shape[0]
    pos = np.arange(t) if pos is None else np.asarray(pos)
    nh, d = mc["heads"], mc["dim"]
    g, dv = mc.get("kv_heads", nh), mc.get("vdim", d)
    q = rms((h @ _np(w[pre + "q"]).T).reshape(t, nh, d), eps) * _np(w[pre + "q.norm"])
    k = rms((h @ _np(w[pre + "k"]).T).reshape(t, g, d), eps) * _np(w[pre + "k.norm"])
    v = (h @ _np(w[pre + "v"]).T).reshape(t, g, dv)
    gate = sigmoid(h @ _np(w[pre + "g"]).T)
    o = np.zeros((t, nh, dv))
    weights = np.zeros((nh, t, t))
    for a in range(nh):
        kv = a // (nh // g)
        oa, weights[a] = _softmax_attend(q[:, a], k[:, kv], v[:, kv], mc["scale"], mc.get("mask"), pos)
        o[:, a] = oa * gate[:, a:a + 1]
    out = o.reshape(t, nh * dv) @ _np(w[pre + "o"]).T
    return (out, weights) if return_weights else out


def expert(w, pre, h):
    a = np.maximum(h @ _np(w[pre + "up"]).T, 0.0)
    return (a * a) @ _np(w[pre + "down"]).T


def route(w, pre, fc, h):
    """Per token: the chosen experts (identity experts are numbered after the real ones) and their weights."""
    rc = fc["router"]
    z = h @ _np(w[pre + "router"]).T
    e = np.exp(z - z.max(-1, keepdims=True))
    s = e / e.sum(-1, keepdims=True)
    choice = s + _np(w[pre + "correction"]) if pre + "correction" in w else s.copy()
    n = z.shape[1]
    gr = rc.get("groups")
    if gr:
        per = n // gr["count"]
        for i in range(h.shape[0]):
            score = [choice[i, a * per:(a + 1) * per].max() for a in range(gr["count"])]
            best = sorted(range(gr["count"]), key=lambda a: (-score[a], a))[:gr["keep"]]
            for a in range(gr["count"]):
                if a not in best:
                    choice[i, a * per:(a + 1) * per] = -np.inf
    order = np.argsort(-choice, axis=-1, kind="stable")[:, :rc["top"]]
    return order, np.take_along_axis(s, order, -1)


def moe(w, pre, fc, h):
    chosen, weight = route(w, pre, fc, h)
    real = fc["router"]["experts"]
    out = np.zeros_like(h)
    for i in range(h.shape[0]):
        for e, s in zip(chosen[i], weight[i]):
            out[i] += s * (expert(w, f"{pre}e{e}.", h[i][None])[0] if e < real else h[i])
    if fc.get("shared"):
        out += expert(w, pre + "shared.", h)
    return out


MIXERS = {"latent_attention": latent_attention, "attention": attention}


def layer_runs(cfg):
    """Layer index of every layer run, in order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, w, tokens, pos=None):
    """Logits ``[t, vocab]`` and the sum of the streams after every layer run ``[runs, t, width]``."""
    eps = cfg["norm"]["eps"]
    x0 = _np(w["embed"])[np.asarray(tokens)]
    ns = int(cfg.get("streams") or 1)
    xs = [x0.copy() for _ in range(ns)]
    hidden = []
    for i in layer_runs(cfg):
        lc = cfg["layers"][i]
        p = f"l{i}."
        for q, has in ((1, True), (2, lc.get("mlp") is not None)):
            if not has:
                continue
            hc = f"{p}hc{q}."
            if hc + "in" in w:
                a, b, c = _np(w[hc + "in"]), _np(w[hc + "mix"]), _np(w[hc + "out"])
            else:
                a, b, c = np.ones(ns), np.eye(ns), np.ones(ns)
            u = sum(a[s] * xs[s] for s in range(ns))
            h = rms(u, eps) * _np(w[f"{p}norm{q}"])
            if q == 1:
                y = MIXERS[lc["type"]](w, p + "mix.", lc["mixer"], h, eps, pos)
            else:
                y = moe(w, p + "mlp.", lc["mlp"], h)
            xs = [sum(b[s, t] * xs[s] for s in range(ns)) + c[t] * y for t in range(ns)]
        hidden.append(sum(xs))
    x = sum(xs)
    logits = (rms(x, eps) * _np(w["final.norm"])) @ _np(w["head"]).T
    return logits, np.stack(hidden)
