"""Ops of the hybrid sequence-mixer stack (``csrc/hybrid`` -> ``jax_llama_amd._C_hybrid``).

Same dispatch rule as the rest of ``ops``: GPU tensors run the hand-written gfx950 kernels (a missing extension
raises), CPU tensors run the PyTorch implementation below (the test / oracle path of the framework).

Conventions: activations between ops are fp32 in both number formats. A weight (or cache) tensor's dtype selects the
arithmetic: bf16 weights -> operands rounded to bf16, fp32 accumulation; fp32 weights -> exact fp32 products.

Mechanisms (each with its constants as arguments, usable by any model of the registry):
  * ``linear`` / ``moe_table``: row-major weights of any shape; a token-id -> experts table routes a mixture of SwiGLU
    experts without a router (expert-grouped GEMM over a counting-sorted batch, or per-row GEMVs for decode);
  * ``norm_residual_``: RMS norm on a sublayer's OUTPUT (scalar or vector gain) fused with the residual add;
  * ``attn_prep`` / ``attn_bias``: per-head RMS-normed q / k / v, position-dependent query temperature, soft-capped
    scores, learned per-distance bias (any bucketing: the table is expanded by distance on the host), causal softmax;
  * ``delta_prep`` / ``delta_scan`` / ``gated_rmsnorm``: the gated delta rule with short causal convolutions;
  * ``latent_prep`` / ``heads_linear`` + ``attn_bias(sink=...)``: latent attention -- one normed low-rank vector per
    token is cached, queries are mapped into the latent space per head, every head attends over the shared latent
    (keys = values = the cache) with a learned sink in the softmax denominator, and the result is mapped out per head;
  * ``linear(act=...)``: squared-ReLU and clamped gated epilogues; ``moe_routed``: a sigmoid-score top-k router whose
    weights scale the experts' INPUTS, plus a gated shared expert (``norm_residual_(extra=...)``);
  * ``rope_prep`` / ``rotate_heads`` + ``attn_bias(chunk=..., head_scale=...)``: projection biases, rotary positions
    on part of each q / k head, values rotated by their own position before caching and the summed values turned
    back by the query's, block-local causal masks, a learned temperature per head;
  * ``mlstm_prep`` / ``mlstm_scan`` and ``token_shift`` / ``timemix_scan``: two linear recurrences over a carried fp32
    matrix state (a stabilised exponential-gate memory with a normaliser; a per-channel-decay memory with a bonus
    for the current token), one scan kernel; ``gated_rmsnorm`` takes either's read-out;
  * ``linear(act=ACT_SOFTCAP)`` and ``linear_add_``: ``cap * tanh(y / cap)`` epilogue; residual add in the epilogue;
  * ``attn_bias(window=, keep_first=, gate=, vdim=)``: sliding-window masks that may keep a sequence's first keys, a
    sigmoid gate per (token, head) on the output, values that are the leading columns of the key rows;
    ``attn_prep(q_w=, k_w=, norm_v=)``: weighted per-head q / k norms; ``latent_rope_prep`` + ``rotate_heads(offset=,
    interleaved=)``: latent attention with a normed query latent and one rotated key part shared by all heads;
  * ``route_grouped`` / ``moe_grouped``: softmax-score router with a selection bias, expert groups and identity
    experts; ``hc_in`` / ``hc_update_``: several residual streams mixed around every sublayer (hyper-connections).
"""
from __future__ import annotations

import importlib
import math
import os
from typing import Optional, Tuple

import torch

BF16 = torch.bfloat16
F32 = torch.float32

# widest value head, and widest key head, the attention kernels take (csrc/hybrid/attn_bias.hip AB_MAX_VREG, AB_MAX_DIM)
ATTN_MAX_HEAD = 512
ATTN_MAX_KEY = 1024
# epilogues of a row linear (csrc/hybrid/hybrid.h RowAct)
ACT_NONE, ACT_RELU2, ACT_SWIGLU, ACT_CLAMP_GLU, ACT_SOFTCAP = 0, 1, 2, 3, 4

_EXT = None
_ERR: Optional[BaseException] = None
# bf16 prefill attention on the MFMA flash kernel where its shapes apply (JLA_HY_MMA_PREFILL=0: the plain kernel, A/B)
MMA_PREFILL = os.environ.get("JLA_HY_MMA_PREFILL", "1") != "0"


def ext():
    """The native module, or a loud error saying how to build it."""
    global _EXT, _ERR
    if _EXT is None and _ERR is None:
        try:
            _EXT = importlib.import_module("jax_llama_amd._C_hybrid")
        except BaseException as e:  # ImportError, OSError (undefined symbol), ...
            _ERR = e
    if _EXT is None:
        raise RuntimeError("jax_llama_amd hybrid HIP extension is not available "
                           f"({type(_ERR).__name__}: {_ERR}). Build it with `python build.py --only hybrid` "
                           "(requires hipcc, targets gfx950). GPU tensors are never run on a fallback path.")
    return _EXT


def ext_available() -> bool:
    try:
        ext()
        return True
    except RuntimeError:
        return False


def so_path() -> Optional[str]:
    return getattr(ext(), "__file__", None) if ext_available() else None


def _gpu(t: torch.Tensor) -> bool:
    return t.device.type == "cuda"


def _slot_tensor(slot, device) -> torch.Tensor:
    if torch.is_tensor(slot):
        return slot
    return torch.tensor([int(slot)], dtype=torch.int32, device=device)


def _slot_int(slot) -> int:
    return int(slot.reshape(-1)[0].item()) if torch.is_tensor(slot) else int(slot)


def _round_like(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """The operand rounding of a product with weight ``w`` (CPU path)."""
    return x.to(BF16).float() if w.dtype == BF16 else x.float()


# ------------------------------------------------------------------------------------------------ rows
def embed_rows(ids: torch.Tensor, table: torch.Tensor, col0: int = 0, ncols: Optional[int] = None,
               scale: float = 1.0, copies: int = 1) -> torch.Tensor:
    """fp32 ``[M, ncols]`` = ``table[ids, col0 : col0 + ncols] * scale``; ``copies > 1``: ``[copies, M, ncols]``, the
    same rows ``copies`` times (the residual streams of a hyper-connected stack all start from the embedding)."""
    ncols = table.shape[1] - col0 if ncols is None else ncols
    ids = ids.reshape(-1)
    if not _gpu(table):
        x = table[ids.long(), col0:col0 + ncols].float() * torch.tensor(scale, dtype=F32)
        return x if copies == 1 else x[None].repeat(copies, 1, 1)
    out = torch.empty(copies * ids.numel(), ncols, dtype=F32, device=table.device)
    ext().embed_rows(ids.to(torch.int32).contiguous(), table, int(col0), out, float(scale), int(copies))
    return out if copies == 1 else out.reshape(copies, ids.numel(), ncols)


# Dense bf16 linears of a prompt-sized batch run on the framework's tuned MFMA GEMM (ops.linear over the fragment-
# packed weight layout, csrc/kernels/gemm.hip) when the main extension is built and the shape fits its layout
# (N % 16 == 0, K % 32 == 0); the row-major kernel here serves every other case. JLA_HY_PACKED_GEMM=0: never.
PACKED_GEMM = os.environ.get("JLA_HY_PACKED_GEMM", "1") != "0"
PACKED_GEMM_MIN_M = 256
GROUPED_GEMV_MAX_R = 64  # rows up to which an expert-sorted batch runs the expert-grouped GEMV (csrc: HY_GROUPED_GEMV_MAX_R)
_PACKED = {}


def _packed_weight(w: torch.Tensor):
    """The fragment-packed copy of a dense ``[N, K]`` bf16 weight (made once, kept beside the row-major one)."""
    key = (w.data_ptr(), tuple(w.shape))
    pw = _PACKED.get(key)
    if pw is None or pw[0] is not w:
        from ..models.weights import PackedLinear
        pw = _PACKED[key] = (w, PackedLinear.from_dense(w, w.device))
    return pw[1]


def _use_packed_gemm(x: torch.Tensor, w: torch.Tensor) -> bool:
    if not PACKED_GEMM or w.dtype != BF16 or w.dim() != 2 or x.shape[0] < PACKED_GEMM_MIN_M:
        return False
    if w.shape[0] % 16 or w.shape[1] % 32 or not x.is_contiguous():
        return False
    from . import ext_available as core_available
    return core_available()


class RmsInput:
    """A sublayer's input ``rms_norm(x) * gain`` that is only written out when a consumer needs it in memory: the GEMV
    kernels norm the row they read themselves (``linear`` / ``moe_routed`` take this object in place of a tensor), the
    tile kernels and the CPU path read ``value()``, computed once."""

    def __init__(self, x: torch.Tensor, gain: torch.Tensor, eps: float):
        self.x, self.gain, self.eps = x, gain, float(eps)
        self._value: Optional[torch.Tensor] = None

    @property
    def shape(self):
        return self.x.shape

    def value(self) -> torch.Tensor:
        if self._value is None:
            self._value = rms_rows(self.x, self.gain, self.eps)
        return self._value


# rows up to which a GEMV norms its input itself: every wave repeats the row statistic, which beats a launch of the norm
# kernel for one or two rows and loses to it from eight (measured on a 2048-wide stack: 8 rows 8 % slower fused)
FUSE_NORM_MAX_ROWS = 2


def _fuse_norm(x, rows: int, n: int):
    """``(tensor, gain, eps)`` a dense linear of ``rows`` rows and ``n`` columns reads: the un-normed rows with the
    norm's gain when the GEMV will run it on the GPU, else the normed value."""
    if not isinstance(x, RmsInput):
        return x, None, 0.0
    if (_gpu(x.x) and x._value is None and x.gain.numel() == x.x.shape[1] and rows <= FUSE_NORM_MAX_ROWS
            and ext().dense_is_gemv(rows, n)):
        return x.x, x.gain, x.eps
    return x.value(), None, 0.0


def act_gated(act: int) -> bool:
    return act in (ACT_SWIGLU, ACT_CLAMP_GLU)


def _act_cpu(y: torch.Tensor, act: int, limit: float, alpha: float) -> torch.Tensor:
    """The epilogue of a row linear on its fp32 product ``y`` (gated forms: gate columns, then up columns)."""
    if act == ACT_NONE:
        return y
    if act == ACT_RELU2:
        return torch.relu(y).square()
    if act == ACT_SOFTCAP:
        return limit * torch.tanh(y / limit)
    n = y.shape[-1] // 2
    g, u = y[..., :n], y[..., n:]
    if act == ACT_SWIGLU:
        return torch.nn.functional.silu(g) * u
    g = g.clamp(max=limit)
    return g * torch.sigmoid(alpha * g) * (u.clamp(-limit, limit) + 1.0)


def linear(x, w: torch.Tensor, swiglu: bool = False, act: int = ACT_NONE, limit: float = 0.0,
           alpha: float = 1.0) -> torch.Tensor:
    """``act(x [M, K] (fp32, or an ``RmsInput``) @ w^T)`` -> fp32 ``[M, N]``. ``act``: none, ``ACT_RELU2`` (``max(y, 0)^2``),
    ``ACT_SOFTCAP`` (``limit * tanh(y / limit)``; ``limit = 1`` is a plain tanh), or a gated
    form for which ``w`` is ``[2N, K]`` (gate rows, then up rows): ``ACT_SWIGLU`` (``silu(g) * u``; also
    ``swiglu=True``) or ``ACT_CLAMP_GLU`` (``g' sigmoid(alpha g') (u' + 1)``, ``g' = min(g, limit)``,
    ``u' = clamp(u, -limit, limit)``). ``x`` may be a column-contiguous view with strided rows."""
    if swiglu:
        act = ACT_SWIGLU
    n = w.shape[0] // 2 if act_gated(act) else w.shape[0]
    x, norm_w, norm_eps = _fuse_norm(x, x.shape[0], n)
    if not _gpu(x):
        return _act_cpu(_round_like(x, w) @ w.float().t(), act, limit, alpha)
    if act == ACT_NONE and norm_w is None and _use_packed_gemm(x, w):
        from . import linear as packed_linear
        xb = torch.empty(x.shape, dtype=BF16, device=x.device)
        ext().cast_bf16(x, xb)
        return packed_linear(xb, _packed_weight(w), out_dtype=F32)
    out = torch.empty(x.shape[0], n, dtype=F32, device=x.device)
    ext().linear_rows(x, None, w, out, None, None, None, x.shape[0], int(act), float(limit), float(alpha), None, norm_w,
                      norm_eps)
    return out


def ff_dense(x, w_up: torch.Tensor, w_down: torch.Tensor, act: int = ACT_RELU2) -> torch.Tensor:
    """``act(x @ w_up^T) @ w_down^T`` with a one-accumulator activation. A prompt-sized bf16 batch runs both products on
    the packed MFMA GEMM: it has no such epilogue, so the activation is applied by the kernel that rounds the hidden
    activation to bf16 for the second product (a pass that product needs anyway). Otherwise the row linear with the
    activation in its epilogue."""
    if isinstance(x, RmsInput) and _gpu(w_up) and x.shape[0] >= PACKED_GEMM_MIN_M:
        x = x.value()  # (the packed GEMM takes a normed activation, it does not norm it)
    if (act in (ACT_NONE, ACT_RELU2) and _gpu(w_up) and not isinstance(x, RmsInput) and _use_packed_gemm(x, w_up)
            and w_down.dtype == BF16 and w_down.shape[0] % 16 == 0 and w_down.shape[1] % 32 == 0
            and (x.shape[0] * w_up.shape[0]) % 8 == 0):
        from . import linear as packed_linear
        xb = torch.empty(x.shape, dtype=BF16, device=x.device)
        ext().cast_bf16(x, xb)
        h = packed_linear(xb, _packed_weight(w_up), out_dtype=F32)
        hb = torch.empty(h.shape, dtype=BF16, device=x.device)
        ext().cast_bf16(h, hb, int(act))
        return packed_linear(hb, _packed_weight(w_down), out_dtype=F32)
    return linear(linear(x, w_up, act=act), w_down)


def linear_add_(res: torch.Tensor, x, w: torch.Tensor) -> torch.Tensor:
    """``res [M, N] (fp32) += x [M, K] @ w^T`` in place: a sublayer's output projection with the residual add in its
    epilogue."""
    x, norm_w, norm_eps = _fuse_norm(x, x.shape[0], w.shape[0])
    if not _gpu(x):
        return res.add_(_round_like(x, w) @ w.float().t())
    if norm_w is None and res.is_contiguous() and _use_packed_gemm(x, w):
        from . import linear_residual as packed_linear_residual
        xb = torch.empty(x.shape, dtype=BF16, device=x.device)
        ext().cast_bf16(x, xb)
        return packed_linear_residual(xb, _packed_weight(w), res)
    ext().linear_rows(x, None, w, res, None, None, None, x.shape[0], ACT_NONE, 0.0, 1.0, None, norm_w, norm_eps, 0, True)
    return res


_HEAD_INDEX = {}


def _head_index(m: int, h: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """Index sets that run a per-head linear as an expert-grouped one: linear row ``p = head * m + token`` reads and
    writes row ``token * h + head``; ``offs[head] = head * m``. Made once per (tokens, heads) and kept (a captured
    decode step replays with the same tensors)."""
    key = (m, h, str(device))
    got = _HEAD_INDEX.get(key)
    if got is None:
        if len(_HEAD_INDEX) > 4096:
            _HEAD_INDEX.clear()
        rows = (torch.arange(m, dtype=torch.int32)[None, :] * h + torch.arange(h, dtype=torch.int32)[:, None]).reshape(-1)
        offs = torch.arange(h + 1, dtype=torch.int32) * m
        got = _HEAD_INDEX[key] = (rows.to(device), offs.to(device))
    return got


def heads_linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Per-head linear: ``x [M, H, K]`` (fp32), ``w [H, N, K]`` -> fp32 ``[M, H, N]``, head ``h`` of every token times
    ``w[h]^T``. Runs the expert-grouped row linear with the heads as its experts."""
    m, h, k = x.shape
    n = w.shape[1]
    if not _gpu(x):
        return torch.einsum("mhk,hnk->mhn", _round_like(x, w), w.float())
    x2 = x.reshape(m * h, k)
    out = torch.empty(m * h, n, dtype=F32, device=x.device)
    e = ext()
    if m == 1 and h <= e.GEMV_MAX_R:  # one token: a GEMV per head
        rows, _ = _head_index(1, h, x.device)
        e.linear_rows(x2, None, w, out, None, None, rows, h, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    else:
        rows, offs = _head_index(m, h, x.device)
        e.linear_rows(x2, rows, w, out, rows, offs, None, m * h, ACT_NONE, 0.0, 1.0, None, None, 0.0, m)
    return out.reshape(m, h, n)


# rows (members x tokens) up to which same-shaped projections of different inputs run as one grouped launch
STACKED_MAX_ROWS = 64
_STACK_INDEX = {}


def stacked_linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Same-shaped linears of different inputs in one launch: ``x [E, M, K]`` (fp32, contiguous), ``w [E, N, K]`` ->
    fp32 ``[E, M, N]``, ``out[e] = x[e] @ w[e]^T``. Runs the expert-grouped row linear (member ``e`` = expert ``e``)."""
    e_n, m, k = x.shape
    n = w.shape[1]
    if not _gpu(x):
        return torch.einsum("emk,enk->emn", _round_like(x, w), w.float())
    rows = e_n * m
    out = torch.empty(rows, n, dtype=F32, device=x.device)
    key = (e_n, m, str(x.device))
    idx = _STACK_INDEX.get(key)
    if idx is None:
        if len(_STACK_INDEX) > 1024:
            _STACK_INDEX.clear()
        ar = torch.arange(e_n + 1, dtype=torch.int32)
        idx = _STACK_INDEX[key] = (ar[:e_n].repeat_interleave(m).to(x.device), (ar * m).to(x.device))
    ex = ext()
    if rows <= ex.GEMV_MAX_R:
        ex.linear_rows(x.reshape(rows, k), None, w, out, None, None, idx[0], rows, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    else:
        ex.linear_rows(x.reshape(rows, k), None, w, out, None, idx[1], None, rows, ACT_NONE, 0.0, 1.0, None, None, 0.0, m)
    return out.reshape(e_n, m, n)


def moe_table(x: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, w_gu: torch.Tensor,
              w_down: torch.Tensor) -> torch.Tensor:
    """Mixture of SwiGLU experts chosen by a ``[vocab, top]`` int32 table of the token id (no router).

    ``w_gu [E, 2F, K]`` (gate rows then up rows), ``w_down [E, D, F]``. Returns the chosen experts' outputs, fp32
    ``[M * top, D]`` in (token, choice) order; the caller averages them (``norm_residual_(nsum=top, ysc=1/top)``)."""
    m, top, e_n = x.shape[0], table.shape[1], w_gu.shape[0]
    r = m * top
    ids = ids.reshape(-1)
    if not _gpu(x):
        ex = table[ids.long()].reshape(-1).long()  # [R]
        xr = _round_like(x, w_gu).repeat_interleave(top, 0)
        y = torch.empty(r, w_down.shape[1], dtype=F32)
        f = w_gu.shape[1] // 2
        for e in ex.unique().tolist():
            sel = (ex == e).nonzero().squeeze(1)
            gu = xr[sel] @ w_gu[e].float().t()
            h = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
            y[sel] = _round_like(h, w_down) @ w_down[e].float().t()
        return y
    dev = x.device
    e = ext()
    idx = torch.empty(4 * r + e_n + 1, dtype=torch.int32, device=dev)
    row_expert, row_tok, sort_tok, sort_dst, offs = idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]
    e.route_table(ids.to(torch.int32).contiguous(), table, e_n, row_expert, row_tok, sort_tok, sort_dst, offs)
    y = torch.empty(r, w_down.shape[1], dtype=F32, device=dev)
    bf16_pair = w_gu.dtype == BF16 and r > GROUPED_GEMV_MAX_R and x.is_contiguous() and x.shape[1] % 8 == 0
    h = None if bf16_pair else torch.empty(r, w_gu.shape[1] // 2, dtype=F32, device=dev)
    if r <= e.GEMV_MAX_R:  # decode: one GEMV per (token, choice) row, expert read on the device
        e.linear_rows(x, row_tok, w_gu, h, None, None, row_expert, r, ACT_SWIGLU, 0.0, 1.0, None, None, 0.0)
        e.linear_rows(h, None, w_down, y, None, None, row_expert, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    elif bf16_pair:
        # prompt-sized, bf16: the tiles read a bf16 copy of x and keep the hidden activation bf16 (the operands they
        # would round to anyway), which halves the activation traffic of both products
        xb = torch.empty(x.shape, dtype=BF16, device=dev)
        e.cast_bf16(x, xb)
        hb = torch.empty(r, w_gu.shape[1] // 2, dtype=BF16, device=dev)
        e.linear_rows(xb, sort_tok, w_gu, hb, None, offs, None, r, ACT_SWIGLU, 0.0, 1.0, None, None, 0.0)
        e.linear_rows(hb, None, w_down, y, sort_dst, offs, None, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    else:  # expert-grouped tiles over the sorted rows; the down projection scatters back to (token, choice) order
        e.linear_rows(x, sort_tok, w_gu, h, None, offs, None, r, ACT_SWIGLU, 0.0, 1.0, None, None, 0.0)
        e.linear_rows(h, None, w_down, y, sort_dst, offs, None, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    return y


def route_topk(z: torch.Tensor, experts: int, top: int):
    """Score router over logits ``z [M, >= experts]`` (fp32; only the first ``experts`` columns are read): per token the
    ``top`` largest (ties to the lower index), weight ``sigmoid(z)`` of each chosen expert, not renormalised. Returns
    ``(row_expert [R], row_w [R])`` in (token, choice) order (the GPU path returns its whole index record instead)."""
    zz = z[:, :experts].float()
    order = torch.sort(zz, dim=-1, descending=True, stable=True).indices[:, :top]
    return order.reshape(-1), torch.sigmoid(torch.gather(zz, 1, order)).reshape(-1)


def moe_routed(x, z: torch.Tensor, top: int, w_gu: torch.Tensor, w_down: torch.Tensor,
               act: int = ACT_CLAMP_GLU, limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """Mixture of gated experts chosen by score: the ``top`` largest of ``z [M, >= E]``'s first ``E`` columns per token,
    weights ``s = sigmoid(z)`` (not renormalised), and the weight multiplies the expert's INPUT:
    ``y[m, c] = W_down[e] act(W_gu[e] (s x[m]))``. ``w_gu [E, 2F, K]`` (gate rows then up rows), ``w_down [E, D, F]``.
    Returns fp32 ``[M * top, D]`` in (token, choice) order; the caller sums a token's rows
    (``norm_residual_(nsum=top)``)."""
    m, e_n = x.shape[0], w_gu.shape[0]
    r = m * top
    f = w_gu.shape[1] // 2
    norm_w, norm_eps = None, 0.0
    if isinstance(x, RmsInput):
        if _gpu(x.x) and x._value is None and r <= ext().GEMV_MAX_R:  # per-row GEMVs norm the rows they gather
            x, norm_w, norm_eps = x.x, x.gain, x.eps
        else:
            x = x.value()
    if not _gpu(x):
        ex, wt = route_topk(z, e_n, top)
        xr = _round_like(x.float().repeat_interleave(top, 0) * wt[:, None], w_gu)
        y = torch.empty(r, w_down.shape[1], dtype=F32)
        for e in ex.unique().tolist():
            sel = (ex == e).nonzero().squeeze(1)
            hid = _act_cpu(xr[sel] @ w_gu[e].float().t(), act, limit, alpha)
            y[sel] = _round_like(hid, w_down) @ w_down[e].float().t()
        return y
    dev = x.device
    e = ext()
    idx = torch.empty(4 * r + e_n + 1, dtype=torch.int32, device=dev)
    row_expert, row_tok, sort_tok, sort_dst, offs = idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]
    wts = torch.empty(2 * r, dtype=F32, device=dev)
    row_w, sort_w = wts[:r], wts[r:]
    y = torch.empty(r, w_down.shape[1], dtype=F32, device=dev)
    if r <= e.GEMV_MAX_R:  # decode: one GEMV per (token, choice) row, expert and weight read on the device
        e.route_topk(z, e_n, top, row_expert, row_tok, row_w, None, None, None, None)  # (no sorted order needed)
        h = torch.empty(r, f, dtype=F32, device=dev)
        e.linear_rows(x, row_tok, w_gu, h, None, None, row_expert, r, int(act), float(limit), float(alpha), row_w,
                      norm_w, norm_eps)
        e.linear_rows(h, None, w_down, y, None, None, row_expert, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    else:
        e.route_topk(z, e_n, top, row_expert, row_tok, row_w, sort_tok, sort_dst, sort_w, offs)
        # expert-grouped over the sorted rows: the scaled fp32 activation is rounded while it is staged; with bf16
        # weights the hidden activation is kept bf16 (the operand the down projection would round it to anyway)
        keep_bf16 = w_gu.dtype == BF16 and r > GROUPED_GEMV_MAX_R
        h = torch.empty(r, f, dtype=BF16 if keep_bf16 else F32, device=dev)
        e.linear_rows(x, sort_tok, w_gu, h, None, offs, None, r, int(act), float(limit), float(alpha), sort_w, None, 0.0)
        e.linear_rows(h, None, w_down, y, sort_dst, offs, None, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    return y


def route_grouped(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int = 1, keep: int = 1):
    """Softmax-score router over logits ``z [M, E]`` (fp32): scores ``s = softmax(z)``; the choice is made on
    ``s + correction`` (``correction [E]``, a selection bias that does not enter the weights); the experts form
    ``groups`` equal groups of neighbours, a group's score is its largest choice score, and only experts of the ``keep``
    best groups can be chosen (ties to the lower index everywhere); the ``top`` largest are chosen, weight ``s`` of each
    (not renormalised). Returns ``(row_expert [R], row_w [R])`` in (token, choice) order."""
    zz = z.float()
    m, e_n = zz.shape
    sc = torch.softmax(zz, -1)
    ch = sc + correction.float().reshape(1, -1) if correction is not None else sc.clone()
    if groups > 1:
        per = e_n // groups
        gs = ch.reshape(m, groups, per).max(-1).values
        best = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        allowed = torch.zeros(m, groups, dtype=torch.bool).scatter_(1, best, True)
        ch = ch.masked_fill(~allowed.repeat_interleave(per, 1), float("-inf"))
    order = torch.sort(ch, dim=-1, descending=True, stable=True).indices[:, :top]
    return order.reshape(-1), torch.gather(sc, 1, order).reshape(-1)


def moe_grouped(x: torch.Tensor, z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int,
                w_up: torch.Tensor, w_down: torch.Tensor, act: int = ACT_RELU2):
    """Experts of a ``route_grouped`` mixture: ``z [M, E + I]`` holds the logits of the ``E = w_up.shape[0]`` real
    experts and of ``I`` identity experts behind them (an identity expert returns its input; it has no weights and runs
    no product). ``w_up [E, F, K]``, ``w_down [E, D, F]``, one-accumulator activation ``act``. Returns
    ``(y [M * top, D], row_expert [M * top], row_w [M * top])`` in (token, choice) order: ``y`` rows of real experts hold
    ``W_down act(W_up x)`` unweighted, rows whose expert is ``>= E`` hold nothing (the caller's ``hc_update_`` puts the
    weighted sum together)."""
    m, e_n, e_all = x.shape[0], w_up.shape[0], z.shape[1]
    r = m * top
    if act_gated(act):
        raise ValueError("moe_grouped: one-accumulator activations only")
    if not _gpu(x):
        ex, wt = route_grouped(z, correction, top, groups, keep)
        xr = _round_like(x.float(), w_up).repeat_interleave(top, 0)
        y = torch.zeros(r, w_down.shape[1], dtype=F32)
        for e in ex.unique().tolist():
            if e >= e_n:
                continue
            sel = (ex == e).nonzero().squeeze(1)
            hid = _act_cpu(xr[sel] @ w_up[e].float().t(), act, 0.0, 1.0)
            y[sel] = _round_like(hid, w_down) @ w_down[e].float().t()
        return y, ex.to(torch.int32), wt
    dev = x.device
    e = ext()
    idx = torch.empty(4 * r + e_all + 1, dtype=torch.int32, device=dev)
    row_expert, row_tok, sort_tok, sort_dst, offs = idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]
    wts = torch.empty(2 * r, dtype=F32, device=dev)
    row_w, sort_w = wts[:r], wts[r:]
    y = torch.empty(r, w_down.shape[1], dtype=F32, device=dev)
    f = w_up.shape[1]
    if r <= e.GEMV_MAX_R:  # decode: one GEMV per (token, choice) row; rows of identity experts are skipped on the device
        e.route_grouped(z, correction, e_all, top, groups, keep, row_expert, row_tok, row_w, None, None, None, None)
        h = torch.empty(r, f, dtype=F32, device=dev)
        e.linear_rows(x, row_tok, w_up, h, None, None, row_expert, r, int(act), 0.0, 1.0, None, None, 0.0)
        e.linear_rows(h, None, w_down, y, None, None, row_expert, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    else:
        # expert-grouped over the sorted rows; identity experts sort behind the real ones, past the last offset the
        # linears look at
        e.route_grouped(z, correction, e_all, top, groups, keep, row_expert, row_tok, row_w, sort_tok, sort_dst, sort_w, offs)
        # with bf16 weights the tiles read a bf16 copy of x and keep the hidden activation bf16 (the operands they would
        # round to anyway): half the activation traffic of both products
        keep_bf16 = w_up.dtype == BF16 and r > GROUPED_GEMV_MAX_R
        h = torch.empty(r, f, dtype=BF16 if keep_bf16 else F32, device=dev)
        xa = x
        if keep_bf16 and x.is_contiguous() and x.numel() % 8 == 0:
            xa = torch.empty(x.shape, dtype=BF16, device=dev)
            e.cast_bf16(x, xa)
        e.linear_rows(xa, sort_tok, w_up, h, None, offs, None, r, int(act), 0.0, 1.0, None, None, 0.0)
        e.linear_rows(h, None, w_down, y, sort_dst, offs, None, r, ACT_NONE, 0.0, 1.0, None, None, 0.0)
    return y, row_expert, row_w


def hc_in(xs: torch.Tensor, a: torch.Tensor) -> torch.Tensor:
    """What a sublayer of a hyper-connected stack reads: ``u [M, D] = sum_s a[s] xs[s]`` for the residual streams
    ``xs [S, M, D]`` (fp32) and the read weights ``a [S]`` (fp32)."""
    if not _gpu(xs):
        return torch.einsum("s,smd->md", a.float(), xs.float())
    u = torch.empty(xs.shape[1], xs.shape[2], dtype=F32, device=xs.device)
    ext().hc_update(xs, None, None, None, 1, None, None, 0, None, None, a, u)
    return u


def hc_update_(xs: torch.Tensor, mix: torch.Tensor, out_w: torch.Tensor, y: torch.Tensor, nsum: int = 1,
               row_w: Optional[torch.Tensor] = None, row_expert: Optional[torch.Tensor] = None, n_real: int = 0,
               ident: Optional[torch.Tensor] = None, extra: Optional[torch.Tensor] = None,
               next_in: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """A sublayer's write into the residual streams ``xs [S, M, D]`` (fp32, in place), all streams at once from the old
    ones: ``xs[t] <- sum_s mix[s, t] xs[s] + out_w[t] * v`` with the sublayer's result ``v [M, D]`` put together here:
    ``v[m] = sum_{c < nsum} w_c * y[m * nsum + c] (+ extra[m])``, ``w_c = row_w[m * nsum + c]`` (absent: 1); a row whose
    ``row_expert`` is ``>= n_real`` stands for an identity expert and contributes ``w_c * ident[m]`` instead (its ``y`` row
    is not read). ``next_in [S]``: also returns ``u [M, D] = sum_t next_in[t] xs[t]`` of the NEW streams, the next
    sublayer's input (or, with ones, the residual itself)."""
    s_n, m, d = xs.shape
    if not _gpu(xs):
        v = y.float().reshape(m, nsum, d)
        if row_w is not None:
            wt = row_w.float().reshape(m, nsum)
            if row_expert is not None:
                real = row_expert.reshape(m, nsum) < n_real
                v = (torch.where(real[..., None], v, torch.zeros_like(v)) * (wt * real)[..., None]).sum(1)
                v = v + (wt * ~real).sum(1, keepdim=True) * ident.float()
            else:
                v = (v * wt[..., None]).sum(1)
        else:
            v = v.sum(1)
        if extra is not None:
            v = v + extra.float()
        new = torch.einsum("st,smd->tmd", mix.float(), xs.float()) + out_w.float()[:, None, None] * v[None]
        xs.copy_(new)
        return torch.einsum("s,smd->md", next_in.float(), xs) if next_in is not None else None
    u = torch.empty(m, d, dtype=F32, device=xs.device) if next_in is not None else None
    ext().hc_update(xs, mix, out_w, y, int(nsum), row_w, row_expert, int(n_real), ident, extra, next_in, u)
    return u


def norm_residual_(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float, nsum: int = 1, ysc: float = 1.0,
                   extra: Optional[torch.Tensor] = None, extra_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x += rms_norm(ysc * sum of each token's nsum rows of y [+ sigmoid(extra_gate) * extra]) * w`` in place; ``w``
    one number or ``[D]``. ``extra [M, D]``: one more summand per token (a shared expert's output) with the logit of
    its gate in ``extra_gate [M, 1]`` (a column view is fine; absent: weight 1)."""
    if not _gpu(x):
        v = y.float().reshape(x.shape[0], nsum, -1).sum(1) * ysc
        if extra is not None:
            v = v + (torch.sigmoid(extra_gate.float()) * extra.float() if extra_gate is not None else extra.float())
        x.add_(v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float().reshape(-1))
        return x
    ext().norm_residual(y, int(nsum), float(ysc), w.reshape(-1), float(eps), x, None, extra, extra_gate)
    return x


def rms_rows(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``y / sqrt(mean(y^2) + eps) * w`` (fp32), ``w`` one number or ``[D]``."""
    if not _gpu(y):
        v = y.float()
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float().reshape(-1)
    out = torch.empty_like(y)
    ext().norm_residual(y, 1, 1.0, w.reshape(-1), float(eps), None, out, None, None)
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place (fp32, contiguous; ``cap = 1``: a tanh)."""
    if not _gpu(x):
        return x.copy_(cap * torch.tanh(x.float() / cap))
    ext().softcap(x, float(cap))
    return x


def linear_softcap(x, w: torch.Tensor, cap: float) -> torch.Tensor:
    """``cap * tanh((x @ w^T) / cap)``: in the linear's epilogue, or, where a prompt-sized product runs on the packed MFMA
    GEMM (which has no such epilogue), as one elementwise pass behind it: a product with a few dozen output columns is
    a handful of tiles for the row-major kernel and a split-K plan for the packed one."""
    if _gpu(w) and not isinstance(x, RmsInput) and _use_packed_gemm(x, w):
        return softcap_(linear(x, w), cap)
    return linear(x, w, act=ACT_SOFTCAP, limit=cap)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def gelu_gate_rows(gp: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """``gelu_tanh(gp) * table[ids, col0 : col0 + D]``."""
    ids = ids.reshape(-1)
    if not _gpu(gp):
        return gelu_tanh(gp.float()) * table[ids.long(), col0:col0 + gp.shape[1]].float()
    g = torch.empty_like(gp)
    ext().gelu_gate_rows(gp, ids.to(torch.int32).contiguous(), table, int(col0), g)
    return g


# ------------------------------------------------------------------------------------------------ attention
def distance_bias_table(rel: torch.Tensor, bias_max: int) -> torch.Tensor:
    """Expand a bucketed ``[buckets, H]`` bias into a per-distance table ``[bias_max + 1, H]`` (fp32; distances past
    the end use the last row). Buckets: the first half one per distance, the second half log-spaced up to
    ``bias_max``: ``bucket(n) = n`` for ``n < B/2``, else ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) * (B - B/2)))``."""
    nb = rel.shape[0]
    half = nb // 2
    rows = []
    for n in range(int(bias_max) + 1):
        if n < half:
            rows.append(n)
        elif half == 0 or bias_max <= half:
            rows.append(nb - 1)
        else:
            rows.append(min(nb - 1, half + int(math.floor(math.log(n / half) / math.log(bias_max / half) * (nb - half)))))
    idx = torch.tensor(rows, dtype=torch.long, device=rel.device)
    return rel.float()[idx].contiguous()


def attn_prep(proj: torch.Tensor, positions: torch.Tensor, slot, b: int, s: int, heads: int, kv_heads: int, dim: int,
              vdim: int, kc: Optional[torch.Tensor], vc: Optional[torch.Tensor], eps: float, temp_coef: float = 0.0,
              temp_every: int = 1, q_w: Optional[torch.Tensor] = None, k_w: Optional[torch.Tensor] = None,
              norm_v: bool = True) -> torch.Tensor:
    """From the fused projection ``proj [B*S, H*dim (+ G*dim + G*vdim) (+ more)]``: q / k divided by their per-head RMS
    over ``dim`` (times the gain ``q_w`` / ``k_w [dim]``, shared by all heads, when given), v over ``vdim``
    (``norm_v=False``: v as projected), q scaled by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``, k / v
    written into the caches ``[B, G, T, .]`` at ``slot + s``. ``kc is None``: the layer reads another layer's cache (q
    only). Returns q ``[B, S, H, dim]`` fp32."""
    m = b * s
    if not _gpu(proj):
        s0 = _slot_int(slot)
        q = proj[:, :heads * dim].float().reshape(m, heads, dim)
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
        if q_w is not None:
            q = q * q_w.float()
        if temp_coef:
            p = positions.reshape(-1).to(torch.int64)
            q = q * (1.0 + temp_coef * torch.log(torch.div(p + 1, temp_every, rounding_mode="floor").float() + 1.0)
                     )[:, None, None]
        if kc is not None:
            k = proj[:, heads * dim:(heads + kv_heads) * dim].float().reshape(b, s, kv_heads, dim)
            v = proj[:, (heads + kv_heads) * dim:(heads + kv_heads) * dim + kv_heads * vdim].float().reshape(
                b, s, kv_heads, vdim)
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
            if k_w is not None:
                k = k * k_w.float()
            if norm_v:
                v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
            kc[:, :, s0:s0 + s] = k.permute(0, 2, 1, 3).to(kc.dtype)
            vc[:, :, s0:s0 + s] = v.permute(0, 2, 1, 3).to(vc.dtype)
        return q.reshape(b, s, heads, dim)
    q = torch.empty(b, s, heads, dim, dtype=F32, device=proj.device)
    ext().attn_prep(proj, positions.reshape(-1).to(torch.int32).contiguous(), _slot_tensor(slot, proj.device), b, s,
                    heads, kv_heads, dim, vdim, kc, vc, q, float(eps), float(temp_coef), int(temp_every), q_w, k_w,
                    bool(norm_v))
    return q


def latent_prep(proj: torch.Tensor, col0: int, w: torch.Tensor, slot, b: int, s: int, cache: torch.Tensor,
                eps: float, q_cols: int = 0) -> Optional[torch.Tensor]:
    """The cached vector of latent attention: columns ``[col0, col0 + rank)`` of ``proj [B*S, .]`` divided by their
    root mean square (``eps`` inside the root), times the plain gain ``w [rank]``, written into ``cache [B, 1, T, rank]``
    at ``slot + s`` (rounded to the cache's type). ``q_cols``: also returns a dense copy of ``proj[:, :q_cols]`` (the
    queries of the same fused projection)."""
    rank = cache.shape[3]
    if not _gpu(proj):
        s0 = _slot_int(slot)
        c = proj[:, col0:col0 + rank].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        cache[:, 0, s0:s0 + s] = c.reshape(b, s, rank).to(cache.dtype)
        return proj[:, :q_cols].contiguous() if q_cols else None
    q = torch.empty(b * s, q_cols, dtype=F32, device=proj.device) if q_cols else None
    ext().latent_prep(proj, int(col0), w, _slot_tensor(slot, proj.device), b, s, cache, float(eps), q, 0, None, None, None)
    return q


def latent_rope_prep(proj: torch.Tensor, q_col0: int, q_w: torch.Tensor, c_col0: int, c_w: torch.Tensor,
                     freq: Optional[torch.Tensor], positions: torch.Tensor, slot, b: int, s: int, cache: torch.Tensor,
                     eps: float) -> torch.Tensor:
    """The step after the fused down projection of a latent attention whose queries go through a latent too and whose
    keys carry one rotated part shared by all heads. From ``proj [B*S, .]``:
      * columns ``[q_col0, q_col0 + len(q_w))``: RMS-normed, times the plain gain ``q_w`` -> returned dense (fp32), the
        input of the queries' up projection;
      * columns ``[c_col0, c_col0 + rank)``, ``rank = len(c_w)``: RMS-normed, times ``c_w`` -> ``cache[b, 0, slot + s, :rank]``;
      * the next ``cache.shape[3] - rank`` columns (not normed): their first ``2 len(freq)`` numbers rotated by the
        token's position, number ``2i`` with number ``2i + 1``, angle ``position * freq[i]`` -> ``cache[..., rank:]``."""
    rank, q_rank = c_w.numel(), q_w.numel()
    nrot = cache.shape[3] - rank
    if not _gpu(proj):
        s0 = _slot_int(slot)
        cq = proj[:, q_col0:q_col0 + q_rank].float()
        cq = cq * torch.rsqrt(cq.pow(2).mean(-1, keepdim=True) + eps) * q_w.float()
        c = proj[:, c_col0:c_col0 + rank].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * c_w.float()
        cache[:, 0, s0:s0 + s, :rank] = c.reshape(b, s, rank).to(cache.dtype)
        if nrot:
            r = proj[:, c_col0 + rank:c_col0 + rank + nrot].float().reshape(b * s, 1, nrot)
            if freq is not None:
                r = _turn_pairs_cpu(r, positions.reshape(-1), freq)
            cache[:, 0, s0:s0 + s, rank:] = r.reshape(b, s, nrot).to(cache.dtype)
        return cq.contiguous()
    cq = torch.empty(b * s, q_rank, dtype=F32, device=proj.device)
    ext().latent_prep(proj, int(c_col0), c_w, _slot_tensor(slot, proj.device), b, s, cache, float(eps), cq, int(q_col0), q_w,
                      freq, positions.reshape(-1).to(torch.int32).contiguous())
    return cq


def latent_expand(cache: torch.Tensor, n: int, w: torch.Tensor, first: int = 0) -> torch.Tensor:
    """Per-head linear maps of the cached latents of slots ``[first, n)``: ``cache [B, 1, T, rank]``, ``w [H, N, rank]``
    -> ``[B, H, n - first, N]`` in the cache's type (the layout of a key / value cache of ``H`` heads whose slot 0 is the
    cache's slot ``first``, so the attention kernels take it as one). Runs the expert-grouped row linear with the heads as
    its experts."""
    b, _, t, rank = cache.shape
    h, nn = w.shape[0], w.shape[1]
    if not _gpu(cache):
        y = torch.einsum("btr,hnr->bhtn", cache[:, 0, first:n].float(), w.float())
        return y.to(cache.dtype)
    dev = cache.device
    if cache.dtype == F32 and w.dtype == BF16:
        raise ValueError("latent_expand: an fp32 cache needs fp32 maps")
    cnt = n - first
    out = torch.empty(b, h, cnt, nn, dtype=cache.dtype, device=dev)
    a_idx, dst, offs = _expand_index(b, t, cnt, h, dev)
    src = cache.reshape(b * t, rank)[first:] if first else cache.reshape(b * t, rank)
    ext().linear_rows(src, a_idx, w, out.reshape(b * h * cnt, nn), dst, offs, None, b * h * cnt,
                      ACT_NONE, 0.0, 1.0, None, None, 0.0)
    return out


_EXPAND_INDEX = {}


def _expand_index(b: int, t: int, n: int, h: int, device):
    """Index sets of ``latent_expand``: linear row ``p = head * (B n) + row * n + token`` reads cache row
    ``row * T + token`` and writes output row ``(row * H + head) * n + token``; ``offs[head] = head * B n``. Kept per
    shape (the keys and the values of every layer of a step ask for the same sets)."""
    key = (b, t, n, h, str(device))
    got = _EXPAND_INDEX.get(key)
    if got is None:
        if len(_EXPAND_INDEX) > 256:
            _EXPAND_INDEX.clear()
        ar = lambda k: torch.arange(k, dtype=torch.int32)  # noqa: E731
        src = (ar(b)[:, None] * t + ar(n)[None, :]).reshape(-1)
        dst = ((ar(b)[None, :, None] * h + ar(h)[:, None, None]) * n + ar(n)[None, None, :]).reshape(-1)
        got = _EXPAND_INDEX[key] = (src.repeat(h).to(device), dst.contiguous().to(device), (ar(h + 1) * (b * n)).to(device))
    return got


def attn_bias(q: torch.Tensor, kc: torch.Tensor, vc: torch.Tensor, slot, scale: float, softcap: float = 0.0,
              bias: Optional[torch.Tensor] = None, max_kv: Optional[int] = None,
              sink: Optional[torch.Tensor] = None, chunk: int = 0,
              head_scale: Optional[torch.Tensor] = None, window: int = 0, keep_first: int = 0,
              gate: Optional[torch.Tensor] = None, vdim: Optional[int] = None) -> torch.Tensor:
    """Causal attention of ``q [B, S, H, dim]`` (queries at cache slots ``slot + s``) over ``[B, G, T, .]`` caches:
    ``score = q.k * scale``; ``softcap * tanh(score / softcap)`` if ``softcap > 0``; ``+ bias[min(i - j, last), h]``;
    softmax over ``j <= i``, with ``exp(sink[h])`` added to the denominator when ``sink [H]`` is given (a slot without
    key or value). ``chunk > 0``: query ``i`` only sees the keys of its own block of ``chunk`` cache slots,
    ``floor(j / chunk) == floor(i / chunk)`` (blocks count from slot 0 of the row, wherever a prompt was cut).
    ``head_scale [H]``: the score of head ``h`` is also multiplied by ``head_scale[h]`` (before cap and bias).
    ``window > 0``: query ``i`` sees key ``j <= i`` only if ``i - j < window`` or ``j < keep_first`` (the first
    ``keep_first`` slots of a row stay visible to every later query). ``gate [B*S, >= H]`` (a column view is fine): head
    ``h``'s output of token ``m`` is multiplied by ``sigmoid(gate[m, h])``. ``kc`` and ``vc`` may be one tensor (latent
    attention); ``vdim``: the values are the first ``vdim`` columns of ``vc``'s rows. Returns fp32 ``[B*S, H*vdim]``."""
    b, s, h, dim = q.shape
    g = kc.shape[1]
    vdim = vc.shape[3] if vdim is None else int(vdim)
    if chunk and window:
        raise ValueError("attn_bias: a block-local mask and a sliding window exclude each other")
    if not _gpu(q):
        s0 = _slot_int(slot)
        t = s0 + s
        k = kc[:, :, :t].float().repeat_interleave(h // g, 1)  # [B, H, t, dim]
        v = vc[:, :, :t, :vdim].float().repeat_interleave(h // g, 1)
        sc = torch.einsum("bshd,bhtd->bhst", q.float(), k) * scale
        if head_scale is not None:
            sc = sc * head_scale.float().reshape(1, h, 1, 1)
        if softcap and softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        qi = torch.arange(s0, t)[:, None]
        kj = torch.arange(t)[None, :]
        dist = qi - kj
        if bias is not None:
            bt = bias.float()[dist.clamp(0, bias.shape[0] - 1)]  # [s, t, H]
            sc = sc + bt.permute(2, 0, 1)[None]
        hidden = dist < 0
        if chunk and chunk > 0:
            hidden = hidden | (torch.div(qi, chunk, rounding_mode="floor") != torch.div(kj, chunk, rounding_mode="floor"))
        if window and window > 0:
            hidden = hidden | ((dist >= window) & (kj >= keep_first))
        sc = sc.masked_fill(hidden[None, None], float("-inf"))
        if sink is not None:
            sc = torch.cat([sc, sink.float().reshape(1, h, 1, 1).expand(b, h, s, 1)], -1)
            pr = torch.softmax(sc, -1)[..., :-1]
        else:
            pr = torch.softmax(sc, -1)
        o = torch.einsum("bhst,bhtv->bshv", pr, v)
        if gate is not None:
            o = o * torch.sigmoid(gate[:, :h].float()).reshape(b, s, h, 1)
        return o.reshape(b * s, h * vdim)
    out = torch.empty(b * s, h * vdim, dtype=F32, device=q.device)
    e = ext()
    t_cap = int(max_kv) if max_kv is not None else kc.shape[2]
    ws, splits, vt = None, 1, None
    if s == 1:
        seen = min(t_cap, chunk) if chunk and chunk > 0 else (min(t_cap, window + keep_first) if window > 0 else t_cap)
        splits = int(e.attn_decode_splits(b, h, seen))
        ws = torch.empty(b * h * splits * (vdim + 2), dtype=F32, device=q.device)
    elif MMA_PREFILL:
        nb = int(e.attn_prefill_ws_bytes(b, s, g, dim, vdim, kc.shape[2], kc.dtype == BF16)) if vdim == vc.shape[3] else 0
        if nb:  # bf16 caches at the MFMA shapes: the flash kernel over a transposed copy of the values
            vt = torch.empty(nb // 2, dtype=BF16, device=q.device)
    e.attn_bias(q.contiguous(), kc, vc, _slot_tensor(slot, q.device), float(scale), float(softcap or 0.0), bias, out,
                t_cap, ws, splits, vt, sink, int(chunk or 0), head_scale, int(window or 0), int(keep_first or 0), gate,
                vdim)
    return out


# ------------------------------------------------------------------------------------------------ gated delta rule
def delta_prep(proj: torch.Tensor, b: int, s: int, heads: int, kv_heads: int, dim: int, vdim: int,
               conv_w: torch.Tensor, conv_state: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor
               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """From ``proj [B*S, q (G*dim) | k (G*dim) | v (H*vdim) | gate (H*vdim) | b (H) | a (H)]``: the short causal
    convolution (``conv_w [channels, taps]``, last tap = current token; earlier inputs from ``conv_state
    [B, channels, taps-1]``, which is advanced) + SiLU on q, k, v; q, k to unit length per head (``1e-6`` inside the
    root; q also times ``dim^-1/2``); ``beta = sigmoid(b)``; ``decay = exp(-exp(a_log) * softplus(a + dt_bias))``.
    Returns ``(q [M,G,dim], k [M,G,dim], v [M,H,vdim], beta [M,H], decay [M,H])`` fp32."""
    m = b * s
    qk, vv = kv_heads * dim, heads * vdim
    c = 2 * qk + vv
    if not _gpu(proj):
        taps = conv_w.shape[1]
        x = proj[:, :c].float().reshape(b, s, c)
        full = torch.cat([conv_state.float().permute(0, 2, 1), x], 1)  # [B, taps-1+S, C]
        y = torch.zeros(b, s, c)
        for tap in range(taps):
            y = y + full[:, tap:tap + s] * conv_w.float()[:, tap]
        if taps > 1:
            conv_state.copy_(full[:, -(taps - 1):].permute(0, 2, 1))
        y = torch.nn.functional.silu(y).reshape(m, c)
        q = y[:, :qk].reshape(m, kv_heads, dim)
        k = y[:, qk:2 * qk].reshape(m, kv_heads, dim)
        v = y[:, 2 * qk:].reshape(m, heads, vdim)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        gates = proj[:, c + vv:c + vv + 2 * heads].float()
        beta = torch.sigmoid(gates[:, :heads])
        decay = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(gates[:, heads:] + dt_bias.float()))
        return q.contiguous(), k.contiguous(), v.contiguous(), beta.contiguous(), decay.contiguous()
    dev = proj.device
    q = torch.empty(m, kv_heads, dim, dtype=F32, device=dev)
    k = torch.empty(m, kv_heads, dim, dtype=F32, device=dev)
    v = torch.empty(m, heads, vdim, dtype=F32, device=dev)
    beta = torch.empty(m, heads, dtype=F32, device=dev)
    decay = torch.empty(m, heads, dtype=F32, device=dev)
    e = ext()
    e.delta_prep(proj, b, s, heads, kv_heads, dim, vdim, conv_w, conv_state, a_log, dt_bias, q, k, v, beta, decay)
    e.conv_state_update(proj, b, s, heads, kv_heads, dim, vdim, conv_w, conv_state)
    return q, k, v, beta, decay


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor,
               state: torch.Tensor, b: int, s: int) -> torch.Tensor:
    """The recurrence per head over ``s`` tokens, ``state [B, H, dim, vdim]`` (fp32) read and advanced in place:
    ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``. Returns ``o [M, H, vdim]``."""
    m, g, dim = q.shape
    h, vdim = v.shape[1], v.shape[2]
    if not _gpu(q):
        rep = h // g
        qq = q.reshape(b, s, g, dim).repeat_interleave(rep, 2)
        kk = k.reshape(b, s, g, dim).repeat_interleave(rep, 2)
        vv = v.reshape(b, s, h, vdim)
        be, de = beta.reshape(b, s, h), decay.reshape(b, s, h)
        o = torch.empty(b, s, h, vdim)
        st = state
        for t in range(s):
            st.mul_(de[:, t, :, None, None])
            u = be[:, t, :, None] * (vv[:, t] - torch.einsum("bhdv,bhd->bhv", st, kk[:, t]))
            st.add_(kk[:, t, :, :, None] * u[:, :, None, :])
            o[:, t] = torch.einsum("bhdv,bhd->bhv", st, qq[:, t])
        return o.reshape(m, h, vdim)
    o = torch.empty(m, h, vdim, dtype=F32, device=q.device)
    ext().delta_scan(q, k, v, beta, decay, state, o, b, s, h, g, dim, vdim)
    return o


GATE_SILU, GATE_SIGMOID = 0, 1


def gated_rmsnorm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, eps: float, gate_act: int = GATE_SILU,
                  denom_floor: Optional[torch.Tensor] = None, gain: float = 1.0,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``o [M, H, vdim] / rms(o) * w * act(gate [M, H*vdim]) * gain`` -> fp32 ``[M, H*vdim]``. ``w``: ``[vdim]`` (one
    gain vector for every head) or ``[H*vdim]``; ``gate_act``: ``GATE_SILU`` or ``GATE_SIGMOID``. ``denom_floor [M, H]``:
    ``o`` is ``[M, H, vdim + 1]`` whose last column is a normaliser ``z``; the head's first ``vdim`` numbers are divided
    by ``max(|z|, denom_floor) + 1e-6`` before the norm. ``out``: a ``[M, H*vdim]`` column slice of a wider buffer."""
    m, h, ov = o.shape
    vdim = ov - 1 if denom_floor is not None else ov
    if out is None:
        out = torch.empty(m, h * vdim, dtype=F32, device=o.device)
    if not _gpu(o):
        x = o.float()
        if denom_floor is not None:
            x = x[..., :vdim] / (torch.maximum(x[..., vdim].abs(), denom_floor.float().reshape(m, h)) + 1e-6)[..., None]
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        x = x.reshape(m, h * vdim) * (w.float().repeat(h) if w.numel() == vdim and h > 1 else w.float().reshape(-1))
        g = gate.float()
        out.copy_(x * (torch.sigmoid(g) if gate_act == GATE_SIGMOID else torch.nn.functional.silu(g)) * gain)
        return out
    ext().gated_rmsnorm(o, gate, w, float(eps), out, h, vdim, int(gate_act), denom_floor, float(gain))
    return out


# ------------------------------------------------------------------------------------------------ rotary positions
def rotary_freqs(base: float, dims: int, device) -> torch.Tensor:
    """float64 ``[dims / 2]``: ``base^(-2 i / dims)``, the turn per position of pair ``i``. Angles are formed in 64-bit
    (position times this) so that a position in the thousands keeps the sine's and cosine's full 32-bit accuracy."""
    if dims < 0 or dims % 2:
        raise ValueError(f"rotary dims must be even, got {dims}")
    return torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64, device=device)


def _turn_cpu(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, sign: float = 1.0) -> torch.Tensor:
    """Rotate the first ``2 len(freq)`` numbers of the last axis of ``x [M, heads, n]`` by ``sign * pos[m]``: number
    ``i`` pairs with ``i + len(freq)``."""
    half = freq.numel()
    if half == 0:
        return x
    ang = pos.reshape(-1).double()[:, None] * freq.double()[None, :] * sign
    c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def _turn_pairs_cpu(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, sign: float = 1.0) -> torch.Tensor:
    """Rotate the first ``2 len(freq)`` numbers of the last axis of ``x [M, heads, n]`` by ``sign * pos[m]``: number
    ``2i`` pairs with number ``2i + 1``."""
    half = freq.numel()
    if half == 0:
        return x
    ang = pos.reshape(-1).double()[:, None] * freq.double()[None, :] * sign
    c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
    u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
    turned = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
    return torch.cat([turned, x[..., 2 * half:]], -1)


def rope_prep(proj: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor, slot, b: int, s: int, heads: int,
              kv_heads: int, dim: int, vdim: int, kc: torch.Tensor, vc: torch.Tensor, qk_freq: torch.Tensor,
              v_freq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From the fused projection ``proj [B*S, H*dim + G*dim + G*vdim]`` (+ ``bias``, one number per column): q and k
    heads rotated by the token's position on their first ``2 len(qk_freq)`` numbers (number ``i`` with
    ``i + len(qk_freq)``, angle ``position * qk_freq[i]``; the rest pass), v heads rotated the same way over
    ``2 len(v_freq)`` numbers when ``v_freq`` is given; k / v written into the caches ``[B, G, T, .]`` at ``slot + s``.
    Returns q ``[B, S, H, dim]`` fp32."""
    m = b * s
    if not _gpu(proj):
        s0 = _slot_int(slot)
        y = proj.float()
        if bias is not None:
            y = y + bias.float()
        pos = positions.reshape(-1)
        q = _turn_cpu(y[:, :heads * dim].reshape(m, heads, dim), pos, qk_freq)
        k = _turn_cpu(y[:, heads * dim:(heads + kv_heads) * dim].reshape(m, kv_heads, dim), pos, qk_freq)
        v = y[:, (heads + kv_heads) * dim:(heads + kv_heads) * dim + kv_heads * vdim].reshape(m, kv_heads, vdim)
        if v_freq is not None:
            v = _turn_cpu(v, pos, v_freq)
        kc[:, :, s0:s0 + s] = k.reshape(b, s, kv_heads, dim).permute(0, 2, 1, 3).to(kc.dtype)
        vc[:, :, s0:s0 + s] = v.reshape(b, s, kv_heads, vdim).permute(0, 2, 1, 3).to(vc.dtype)
        return q.reshape(b, s, heads, dim).contiguous()
    q = torch.empty(b, s, heads, dim, dtype=F32, device=proj.device)
    ext().rope_prep(proj, bias, positions.reshape(-1).to(torch.int32).contiguous(), _slot_tensor(slot, proj.device), b, s,
                    heads, kv_heads, dim, vdim, kc, vc, q, qk_freq, v_freq)
    return q


def rotate_heads(a: torch.Tensor, positions: torch.Tensor, freq: Optional[torch.Tensor], heads: int, sign: float = 1.0,
                 gain: float = 1.0, out: Optional[torch.Tensor] = None, offset: int = 0,
                 interleaved: bool = False) -> torch.Tensor:
    """``out [M, heads * n] = turn(a [M, heads * n], sign * position) * gain``: in every head the ``2 len(freq)`` numbers
    from ``offset`` on are rotated by ``sign`` times the row's position (pairs ``i``, ``i + len(freq)``, or with
    ``interleaved`` pairs ``2i``, ``2i + 1``); ``freq`` None: a scaled copy. ``out`` may be a column slice of a wider
    buffer, or ``a`` itself."""
    m = a.shape[0]
    n = a.shape[1] // heads
    if out is None:
        out = torch.empty(m, heads * n, dtype=F32, device=a.device)
    if not _gpu(a):
        x = a.float().reshape(m, heads, n)
        if freq is not None:
            turn = _turn_pairs_cpu if interleaved else _turn_cpu
            x = torch.cat([x[..., :offset], turn(x[..., offset:], positions.reshape(-1), freq, sign)], -1)
        out.copy_(x.reshape(m, heads * n) * gain)
        return out
    ext().rotate_heads(a, positions.reshape(-1).to(torch.int32).contiguous(), freq, heads, float(sign), float(gain), out,
                       int(offset), bool(interleaved))
    return out


# ------------------------------------------------------------------------------------------------ linear recurrences
def token_shift(h: torch.Tensor, prev: torch.Tensor, mu: torch.Tensor, b: int, s: int) -> torch.Tensor:
    """``out[n, m] = h[m] + (h[m - 1] - h[m]) * mu[n]`` for the ``n`` rows of ``mu [n, D]``; the token before a call's
    first comes from ``prev [B, D]`` (zeros at a sequence start), which is then set to the call's last token. fp32
    ``[n, B*S, D]``."""
    n, d = mu.shape
    if not _gpu(h):
        hh = h.float().reshape(b, s, d)
        before = torch.cat([prev.float()[:, None], hh[:, :-1]], 1)
        out = hh[None] + (before - hh)[None] * mu.float()[:, None, None, :]
        prev.copy_(hh[:, -1])
        return out.reshape(n, b * s, d).contiguous()
    out = torch.empty(n, b * s, d, dtype=F32, device=h.device)
    ext().token_shift(h, prev, mu, out, b, s)
    return out


def mlstm_prep(proj: torch.Tensor, col_i: int, col_f: int, gate_bias: torch.Tensor, cap: float, mstate: torch.Tensor,
               b: int, s: int, heads: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gates of the stabilised exponential-gate memory from columns of ``proj [B*S, .]``: per head
    ``a = cap tanh((proj[col_i + h] + gate_bias[h]) / cap)``, ``f = logsigmoid(cap tanh((proj[col_f + h] +
    gate_bias[H + h]) / cap))``, the running maximum ``m_t = max(f + m_(t-1), a)`` carried in ``mstate [B, H]`` (0 at a
    sequence start; advanced). Returns ``(keep, write, floor)`` fp32 ``[B*S, H]``: ``exp(f + m_(t-1) - m_t)``,
    ``exp(a - m_t)``, ``exp(-m_t)``."""
    m = b * s
    if not _gpu(proj):
        gb = gate_bias.float()
        a = cap * torch.tanh((proj[:, col_i:col_i + heads].float() + gb[:heads]) / cap)
        f = torch.nn.functional.logsigmoid(cap * torch.tanh((proj[:, col_f:col_f + heads].float() + gb[heads:]) / cap))
        a, f = a.reshape(b, s, heads), f.reshape(b, s, heads)
        keep, write, floor = torch.empty(b, s, heads), torch.empty(b, s, heads), torch.empty(b, s, heads)
        mm = mstate.float().clone()
        for t in range(s):
            m_new = torch.maximum(f[:, t] + mm, a[:, t])
            keep[:, t] = torch.exp(f[:, t] + mm - m_new)
            write[:, t] = torch.exp(a[:, t] - m_new)
            floor[:, t] = torch.exp(-m_new)
            mm = m_new
        mstate.copy_(mm)
        return keep.reshape(m, heads), write.reshape(m, heads), floor.reshape(m, heads)
    out = torch.empty(3, m, heads, dtype=F32, device=proj.device)
    ext().mlstm_prep(proj, int(col_i), int(col_f), gate_bias, float(cap), mstate, out, b, s, heads)
    return out[0], out[1], out[2]


# A prompt's recurrence runs as several segments side by side when one pass would leave most of the chip idle: segments
# of at least SCAN_SEG_MIN tokens, as many as bring the launch to about SCAN_TARGET_BLOCKS workgroups.
SCAN_SEG_MIN = 64
SCAN_TARGET_BLOCKS = int(os.environ.get("JLA_HY_SCAN_BLOCKS", "1024"))


def _scan_segments(b: int, s: int, heads: int, dim: int, cols: int, device):
    """``(nseg, seg_len, workspace)`` of a scan over ``s`` tokens of ``b`` rows (csrc/hybrid/recurrent.hip: a thread
    holds 16 key rows of a state column, 256 threads a workgroup)."""
    lanes = 1
    while lanes * 16 < dim:
        lanes *= 2
    blocks = b * heads * ((cols * lanes + 255) // 256)
    nseg = min(s // SCAN_SEG_MIN, SCAN_TARGET_BLOCKS // max(1, blocks))
    if nseg < 2:
        return 1, max(s, 1), None
    seg_len = (s + nseg - 1) // nseg
    nseg = (s + seg_len - 1) // seg_len
    ws = torch.empty(b * nseg * heads * dim * (cols + 1), dtype=F32, device=device)
    return nseg, seg_len, ws


def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, keep: torch.Tensor, write: torch.Tensor,
               state: torch.Tensor, b: int, s: int, q_scale: float = 1.0) -> torch.Tensor:
    """Matrix memory with scalar gates per head, read after the write. ``q, k [M, H, dim]``, ``v [M, H, vdim]`` (column
    views of a projection are fine), ``keep, write [M, H]``; ``state [B, H, dim, vdim + 1]`` (fp32, advanced), whose last
    column is the normaliser (the memory of a value that is always 1):
    ``S <- keep S + write k [v, 1]^T;  o = S^T (q_scale q)``. Returns ``o [M, H, vdim + 1]``."""
    m, h, dim = q.shape
    vdim = v.shape[2]
    if not _gpu(q):
        qq = q.float().reshape(b, s, h, dim) * q_scale
        kk = k.float().reshape(b, s, h, dim)
        vv = torch.cat([v.float().reshape(b, s, h, vdim), torch.ones(b, s, h, 1)], -1)
        ke, wr = keep.float().reshape(b, s, h), write.float().reshape(b, s, h)
        o = torch.empty(b, s, h, vdim + 1)
        for t in range(s):
            state.mul_(ke[:, t, :, None, None])
            state.add_(wr[:, t, :, None, None] * kk[:, t, :, :, None] * vv[:, t, :, None, :])
            o[:, t] = torch.einsum("bhdv,bhd->bhv", state, qq[:, t])
        return o.reshape(m, h, vdim + 1)
    o = torch.empty(m, h, vdim + 1, dtype=F32, device=q.device)
    nseg, seg_len, ws = _scan_segments(b, s, h, dim, vdim + 1, q.device)
    ext().lin_scan(0, q, k, v, keep, write, None, None, state, o, b, s, float(q_scale), nseg, seg_len, ws)
    return o


def timemix_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, wpre: torch.Tensor, w0: torch.Tensor,
                 u: torch.Tensor, state: torch.Tensor, b: int, s: int) -> torch.Tensor:
    """Matrix memory with a decay per key channel and a bonus for the current token, read before the write.
    ``r, k [M, H, dim]``, ``v [M, H, vdim]``, ``wpre [M, H, dim]`` (column views are fine), ``w0, u [H, dim]``;
    ``state [B, H, dim, vdim]`` (fp32, advanced): ``d = exp(-exp(wpre + w0))``;
    ``o = (S + diag(u) k v^T)^T r;  S <- diag(d) S + k v^T``. Returns ``o [M, H, vdim]``."""
    m, h, dim = r.shape
    vdim = v.shape[2]
    if not _gpu(r):
        rr, kk = r.float().reshape(b, s, h, dim), k.float().reshape(b, s, h, dim)
        vv = v.float().reshape(b, s, h, vdim)
        dd = torch.exp(-torch.exp(wpre.float().reshape(b, s, h, dim) + w0.float().reshape(h, dim)))
        uu = u.float().reshape(h, dim)
        o = torch.empty(b, s, h, vdim)
        for t in range(s):
            kv = kk[:, t, :, :, None] * vv[:, t, :, None, :]
            o[:, t] = torch.einsum("bhdv,bhd->bhv", state + uu[None, :, :, None] * kv, rr[:, t])
            state.mul_(dd[:, t, :, :, None])
            state.add_(kv)
        return o.reshape(m, h, vdim)
    o = torch.empty(m, h, vdim, dtype=F32, device=r.device)
    nseg, seg_len, ws = _scan_segments(b, s, h, dim, vdim, r.device)
    ext().lin_scan(1, r, k, v, wpre, None, w0.reshape(h, dim), u.reshape(h, dim), state, o, b, s, 1.0, nseg, seg_len, ws)
    return o
