"""Plain, slow float64 implementation of the Besulix decoder for the tests: one function per mechanism, written from
the equations as token-by-token loops, no cache (a whole sequence is recomputed from its first token) and no code
shared with the package. Inputs: the config as a plain dict (the config.json layout) and a checkpoint-named dict of
tensors.

Notation (x: residual, eps = norm.eps, n(y; w) = y / sqrt(mean(y^2) + eps) * w, t: position from 0):
  embedding   x = n(embed[token]; embed.norm)
  layer       x += mixer(n(x; norm1));  x += ff(n(x; norm2)) when the layer has a feed-forward
  mlstm       q = W_q h / sqrt(dim), k = W_k h, v = W_v h per head; a = cap tanh((W_i h + b_i) / cap),
              f = logsigmoid(cap tanh((W_f h + b_f) / cap)); m_t = max(f + m_(t-1), a) with m_(-1) = 0;
              S_t = e^(f + m_(t-1) - m_t) S_(t-1) + e^(a - m_t) k v^T, z_t the same with k alone;
              o = S_t^T q / (max(|z_t . q|, e^(-m_t)) + 1e-6); y = W_o (concat_h(o / rms(o)) * norm * sigmoid(W_g h))
  parallel    left_scale * attention(h) + right_scale * timemix(h)
  attention   q, k, v = W h + b per head (query head h reads key head h // (H / G)); q, k turned by t on their first
              rot.dims numbers (number i with i + dims / 2, angle t base^(-2 i / dims)); v_j turned by j over all vdim
              numbers the same way; s_ij = q_i . k_j * scale * temp_h for j <= i in the same block of mask.size
              positions; p_ij = e^s_ij / (e^sink_h + sum_j' e^s_ij'); o_i = turn(sum_j p_ij v_j, -i); y = W_o concat(o)
  timemix     x_s = h_t + (h_(t-1) - h_t) mu_s for s in r, k, v, g, w (h_(-1) = 0); r, k, v = W x_s per head,
              gate = silu(W_g x_g), decay d = exp(-exp(W_w2 tanh(W_w1 x_w) + w0)) per head and key channel;
              o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t;  S_t = diag(d_t) S_(t-1) + k_t v_t^T;
              y = W_o (concat_h(o / rms(o)) * norm * gate)
  ff          g = min(W_gate h, limit), u = clip(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))
  logits      z = head n(x; final.norm); cap * tanh(z / cap), cap = logit_softcap
"""
import math

import numpy as np


def _np(t):
    return t.detach().to("cpu").double().numpy() if hasattr(t, "detach") else np.asarray(t, dtype=np.float64)


def rms(y, eps):
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def logsigmoid(z):
    return -np.logaddexp(0.0, -z)


def turn(vec, pos, base, dims):
    """Rotate the first ``dims`` numbers of ``vec`` by position ``pos``: number i pairs with i + dims / 2."""
    out = np.array(vec, dtype=np.float64)
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = vec[i], vec[i + half]
        out[i] = u * c - w * s
        out[i + half] = w * c + u * s
    return out


def chunked_sink_attention(w, pre, mc, h, return_weights=False):
    t = h.shape[0]
    nh, g, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    base, rd, size = mc["rot"]["base"], mc["rot"]["dims"], mc["mask"]["size"]
    q = (h @ _np(w[pre + "q"]).T + _np(w[pre + "q.b"])).reshape(t, nh, d)
    k = (h @ _np(w[pre + "k"]).T + _np(w[pre + "k.b"])).reshape(t, g, d)
    v = (h @ _np(w[pre + "v"]).T + _np(w[pre + "v.b"])).reshape(t, g, dv)
    temp, sink = _np(w[pre + "temp"]), _np(w[pre + "sink"])
    for i in range(t):
        for hd in range(nh):
            q[i, hd] = turn(q[i, hd], i, base, rd)
        for kh in range(g):
            k[i, kh] = turn(k[i, kh], i, base, rd)
            v[i, kh] = turn(v[i, kh], i, base, dv)
    o = np.zeros((t, nh, dv))
    weights = np.zeros((nh, t, t))
    for hd in range(nh):
        kh = hd // (nh // g)
        for i in range(t):
            lo = (i // size) * size
            s = (k[lo:i + 1, kh] @ q[i, hd]) * mc["scale"] * temp[hd]
            m = max(s.max(), sink[hd])
            e = np.exp(s - m)
            p = e / (e.sum() + np.exp(sink[hd] - m))
            weights[hd, i, lo:i + 1] = p
            o[i, hd] = turn(p @ v[lo:i + 1, kh], -i, base, dv)
    out = o.reshape(t, nh * dv) @ _np(w[pre + "o"]).T
    return (out, weights) if return_weights else out


def time_mix(w, pre, mc, h, eps):
    t, width = h.shape
    nh, d = mc["heads"], mc["dim"]
    prev = np.concatenate([np.zeros((1, width)), h[:-1]], 0)

    def mixed(s):
        return h + (prev - h) * _np(w[pre + "mu." + s])

    r = (mixed("r") @ _np(w[pre + "r"]).T).reshape(t, nh, d)
    k = (mixed("k") @ _np(w[pre + "k"]).T).reshape(t, nh, d)
    v = (mixed("v") @ _np(w[pre + "v"]).T).reshape(t, nh, d)
    gz = mixed("g") @ _np(w[pre + "g"]).T
    gate = gz * sigmoid(gz)
    decay = np.exp(-np.exp(np.tanh(mixed("w") @ _np(w[pre + "w1"]).T) @ _np(w[pre + "w2"]).T + _np(w[pre + "w0"])))
    decay = decay.reshape(t, nh, d)
    u = _np(w[pre + "u"]).reshape(nh, d)
    o = np.zeros((t, nh, d))
    for hd in range(nh):
        state = np.zeros((d, d))
        for i in range(t):
            kv = np.outer(k[i, hd], v[i, hd])
            o[i, hd] = (state + u[hd][:, None] * kv).T @ r[i, hd]
            state = decay[i, hd][:, None] * state + kv
    y = rms(o, eps).reshape(t, nh * d) * _np(w[pre + "norm"]) * gate
    return y @ _np(w[pre + "o"]).T


def parallel_mixer(w, pre, mc, h, eps):
    return (mc["left_scale"] * chunked_sink_attention(w, pre + "left.", mc["left"], h)
            + mc["right_scale"] * time_mix(w, pre + "right.", mc["right"], h, eps))


def mlstm(w, pre, mc, h, eps):
    t = h.shape[0]
    nh, d, dv, cap = mc["heads"], mc["dim"], mc["vdim"], mc["gate_cap"]
    q = (h @ _np(w[pre + "q"]).T).reshape(t, nh, d) / math.sqrt(d)
    k = (h @ _np(w[pre + "k"]).T).reshape(t, nh, d)
    v = (h @ _np(w[pre + "v"]).T).reshape(t, nh, dv)
    gi = cap * np.tanh((h @ _np(w[pre + "i"]).T + _np(w[pre + "i.b"])) / cap)
    gf = logsigmoid(cap * np.tanh((h @ _np(w[pre + "f"]).T + _np(w[pre + "f.b"])) / cap))
    o = np.zeros((t, nh, dv))
    for hd in range(nh):
        state, z, m = np.zeros((d, dv)), np.zeros(d), 0.0
        for i in range(t):
            m_new = max(gf[i, hd] + m, gi[i, hd])
            keep, write = math.exp(gf[i, hd] + m - m_new), math.exp(gi[i, hd] - m_new)
            state = keep * state + write * np.outer(k[i, hd], v[i, hd])
            z = keep * z + write * k[i, hd]
            m = m_new
            o[i, hd] = state.T @ q[i, hd] / (max(abs(z @ q[i, hd]), math.exp(-m)) + 1e-6)
    y = rms(o, eps).reshape(t, nh * dv) * _np(w[pre + "norm"]) * sigmoid(h @ _np(w[pre + "g"]).T)
    return y @ _np(w[pre + "o"]).T


def feed_forward(w, pre, fc, h):
    limit = fc["limit"]
    g = np.minimum(h @ _np(w[pre + "gate"]).T, limit)
    u = np.clip(h @ _np(w[pre + "up"]).T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ _np(w[pre + "down"]).T


def forward(cfg, w, tokens):
    """Logits ``[t, vocab]`` and the residual stream after every layer ``[layers, t, width]``."""
    eps = cfg["norm"]["eps"]
    x = rms(_np(w["embed"])[np.asarray(tokens)], eps) * _np(w["embed.norm"])
    hidden = []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps) * _np(w[p + "norm1"])
        if lc["type"] == "mlstm":
            x = x + mlstm(w, p + "mix.", lc["mixer"], h, eps)
        elif lc["type"] == "parallel":
            x = x + parallel_mixer(w, p + "mix.", lc["mixer"], h, eps)
        else:
            raise ValueError(lc["type"])
        if lc.get("mlp") is not None:
            x = x + feed_forward(w, p + "mlp.", lc["mlp"], rms(x, eps) * _np(w[p + "norm2"]))
        hidden.append(x.copy())
    z = (rms(x, eps) * _np(w["final.norm"])) @ _np(w["head"]).T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return z, np.stack(hidden)
