"""Static, pre-allocated KV cache.

Reference: Flax ``"cache"`` collection created by ``init_cache`` (``model.py:459-476``) and
updated by ``_concatenate_to_cache`` (``model.py:169-199``): per layer ``cached_key`` /
``cached_value`` of shape ``(B, T_max, Hkv, Dh)`` holding post-RoPE keys, plus a scalar
``cache_index`` advanced by the number of tokens written.

Here: two tensors ``[L, B, Hkv_local, T_max, Dh]`` (bf16) so that one (b, kv-head)'s keys
are a single contiguous ``T x 256 B`` run — the decode attention kernel streams it with
1 KiB-per-wave-instruction loads — and the slot index is mirrored in a device int32 so
hipGraph-captured decode steps read/advance it without host round trips. No forward pass
is run to create it (unlike the reference's ``module.init`` trick).
"""
from __future__ import annotations

import torch


class KVCache:
    def __init__(self, num_layers: int, batch_size: int, num_kv_heads: int, max_length: int,
                 head_dim: int, device, dtype=torch.bfloat16):
        device = torch.device(device)
        shape = (num_layers, batch_size, num_kv_heads, max_length, head_dim)
        self.k = torch.zeros(shape, dtype=dtype, device=device)
        self.v = torch.zeros(shape, dtype=dtype, device=device)
        self.batch_size = batch_size
        self.max_length = max_length
        self.index = 0  # host mirror of the number of filled slots
        self.index_t = torch.zeros(1, dtype=torch.int32, device=device)

    @property
    def device(self):
        return self.k.device

    def layer(self, i: int):
        return self.k[i], self.v[i]

    def advance(self, n: int) -> None:
        self.index += n
        self.index_t.add_(n)

    def reset(self) -> None:
        self.index = 0
        self.index_t.zero_()

    def clear(self) -> None:
        """``reset`` and zero the keys and values (after a failed step may have left non-finite rows)."""
        self.reset()
        self.k.zero_()
        self.v.zero_()

    def rows(self, b0: int, b1: int) -> "KVCacheRows":
        """The cache of batch rows ``[b0, b1)`` (every layer): a view whose per-layer K / V are contiguous slices, for a
        prefill run in row chunks (runtime/engine.py)."""
        return KVCacheRows(self, b0, b1)

    def nbytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()

    # Flax-cache-like view for API parity / debugging (per-layer dict, (B, T, Hkv, Dh)).
    def as_dict(self):
        return {
            str(i): {
                "cached_key": self.k[i].permute(0, 2, 1, 3),
                "cached_value": self.v[i].permute(0, 2, 1, 3),
                "cache_index": self.index,
            }
            for i in range(self.k.shape[0])
        }


class KVCacheRows:
    """Rows ``[b0, b1)`` of a KVCache: ``layer(i)`` gives contiguous ``[b1 - b0, Hkv, T, Dh]`` views; the slot index is
    the parent's (one position for every row)."""

    def __init__(self, parent: KVCache, b0: int, b1: int):
        self.parent = parent
        self.b0, self.b1 = b0, b1
        self.batch_size = b1 - b0
        self.max_length = parent.max_length

    @property
    def device(self):
        return self.parent.device

    @property
    def index(self):
        return self.parent.index

    @property
    def index_t(self):
        return self.parent.index_t

    def layer(self, i: int):
        return self.parent.k[i, self.b0:self.b1], self.parent.v[i, self.b0:self.b1]


class HybridCache:
    """Per-layer sequence state of a stack that mixes attention and recurrent layers, pre-allocated.

    ``specs[i]`` describes layer ``i``:
      * ``("kv", kv_heads, dim, vdim)``: keys ``[B, G, T, dim]`` and values ``[B, G, T, vdim]`` (head sizes are per
        layer, keys and values may differ in width);
      * ``("latent", rank)``: one vector of ``rank`` numbers per token, ``[B, 1, T, rank]``; ``layer(i)`` returns it as
        both keys and values (every head's keys and values are linear maps of it, applied outside the cache);
      * ``("kv_from", j)``: no storage, ``layer(i)`` is layer ``j``'s keys and values (cross-layer KV sharing);
      * ``("delta", heads, kv_heads, dim, vdim, taps)``: a recurrent state ``[B, H, dim, vdim]`` (always fp32) and
        the short convolutions' input tail ``[B, 2 G dim + H vdim, taps - 1]`` (fp32);
      * ``("mlstm", heads, dim, vdim)``: a matrix memory with its normaliser as one more value column
        ``[B, H, dim, vdim + 1]`` and the running maximum of its gates ``[B, H]`` (fp32);
      * ``("timemix", heads, dim, vdim, width)``: a matrix memory ``[B, H, dim, vdim]`` and the previous token's
        mixer input ``[B, width]`` (fp32);
      * ``("multi", spec, spec, ...)``: a layer whose mixers run side by side, each with its own entry (at most one
        that holds keys and one that is recurrent);
      * ``None``: nothing.
    The slot index (tokens held, the same for every row) is mirrored on the device like ``KVCache``'s, so captured
    decode steps advance it without the host. ``dtype`` is the key / value element type (bf16, or fp32 for exact runs).
    Recurrent state has no slot: ``reset`` zeroes it, since a new sequence starts from a zero state."""

    def __init__(self, specs, batch_size: int, max_length: int, device, dtype=torch.bfloat16):
        device = torch.device(device)
        self.specs = list(specs)
        self.batch_size = batch_size
        self.max_length = max_length
        self.dtype = dtype
        self._k, self._v, self._state, self._conv = {}, {}, {}, {}
        for i, sp in enumerate(self.specs):
            for part in self.parts(sp):
                self._alloc(i, part, batch_size, max_length, dtype, device)
        self._device = device
        self.index = 0
        self.index_t = torch.zeros(1, dtype=torch.int32, device=device)

    @staticmethod
    def parts(sp) -> list:
        """The primitive entries of a layer's spec."""
        if sp is None:
            return []
        if sp[0] == "multi":
            kinds = [p[0] for p in sp[1:]]
            if sum(k in ("kv", "latent", "kv_from") for k in kinds) > 1 or \
                    sum(k in ("delta", "mlstm", "timemix") for k in kinds) > 1:
                raise ValueError(f"a layer holds at most one key / value entry and one recurrent entry: {sp!r}")
            return list(sp[1:])
        return [sp]

    def _alloc(self, i: int, sp, batch_size: int, max_length: int, dtype, device) -> None:
        f32 = dict(dtype=torch.float32, device=device)
        if sp[0] == "kv":
            _, g, dim, vdim = sp
            self._k[i] = torch.zeros(batch_size, g, max_length, dim, dtype=dtype, device=device)
            self._v[i] = torch.zeros(batch_size, g, max_length, vdim, dtype=dtype, device=device)
        elif sp[0] == "latent":
            self._k[i] = self._v[i] = torch.zeros(batch_size, 1, max_length, sp[1], dtype=dtype, device=device)
        elif sp[0] == "kv_from":
            j = sp[1]
            if not (0 <= j < i) or self.specs[j] is None or self.specs[j][0] != "kv":
                raise ValueError(f"layer {i} shares the keys / values of layer {j}, which holds none before it")
        elif sp[0] == "delta":
            _, h, g, dim, vdim, taps = sp
            self._state[i] = torch.zeros(batch_size, h, dim, vdim, **f32)
            self._conv[i] = torch.zeros(batch_size, 2 * g * dim + h * vdim, max(taps - 1, 0), **f32)
        elif sp[0] == "mlstm":
            _, h, dim, vdim = sp
            self._state[i] = torch.zeros(batch_size, h, dim, vdim + 1, **f32)
            self._conv[i] = torch.zeros(batch_size, h, **f32)
        elif sp[0] == "timemix":
            _, h, dim, vdim, width = sp
            self._state[i] = torch.zeros(batch_size, h, dim, vdim, **f32)
            self._conv[i] = torch.zeros(batch_size, width, **f32)
        else:
            raise ValueError(f"unknown cache spec {sp!r}")

    @property
    def device(self):
        return self._device

    def layer(self, i: int):
        """Keys and values layer ``i`` attends over (its own, or the layer's it shares them with)."""
        j = i
        for part in self.parts(self.specs[i]):
            if part[0] == "kv_from":
                j = part[1]
        return self._k[j], self._v[j]

    def owns_kv(self, i: int) -> bool:
        return any(part[0] == "kv" for part in self.parts(self.specs[i]))

    def recurrent(self, i: int):
        """The two carried tensors of a recurrent layer: ``(state, convolution tail)`` (delta), ``(state with the
        normaliser column, running maximum)`` (mlstm) or ``(state, previous token's input)`` (timemix)."""
        return self._state[i], self._conv[i]

    def advance(self, n: int) -> None:
        self.index += n
        self.index_t.add_(n)

    def reset(self) -> None:
        """Empty: slot 0, zero recurrent state (keys and values past the slot are never read)."""
        self.index = 0
        self.index_t.zero_()
        for t in list(self._state.values()) + list(self._conv.values()):
            t.zero_()

    def clear(self) -> None:
        """``reset`` and zero the keys and values too (after a failed step may have left non-finite rows)."""
        self.reset()
        for t in {id(t): t for t in list(self._k.values()) + list(self._v.values())}.values():
            t.zero_()

    def rows(self, b0: int, b1: int) -> "HybridCacheRows":
        return HybridCacheRows(self, b0, b1)

    def nbytes(self) -> int:
        seen = {id(t): t for d in (self._k, self._v, self._state, self._conv) for t in d.values()}
        return sum(t.numel() * t.element_size() for t in seen.values())

    @staticmethod
    def bytes_per(specs, batch_size: int, max_length: int, dtype=torch.bfloat16) -> int:
        """Bytes a cache of this geometry takes (without allocating it)."""
        es = torch.empty(0, dtype=dtype).element_size()
        n = 0
        for layer in specs:
            for sp in HybridCache.parts(layer):
                if sp[0] == "kv":
                    n += batch_size * sp[1] * max_length * (sp[2] + sp[3]) * es
                elif sp[0] == "latent":
                    n += batch_size * max_length * sp[1] * es
                elif sp[0] == "delta":
                    _, h, g, dim, vdim, taps = sp
                    n += 4 * batch_size * (h * dim * vdim + (2 * g * dim + h * vdim) * max(taps - 1, 0))
                elif sp[0] == "mlstm":
                    n += 4 * batch_size * sp[1] * (sp[2] * (sp[3] + 1) + 1)
                elif sp[0] == "timemix":
                    n += 4 * batch_size * (sp[1] * sp[2] * sp[3] + sp[4])
        return n


class HybridCacheRows:
    """Rows ``[b0, b1)`` of a HybridCache (contiguous slices of every tensor; the slot index is the parent's)."""

    def __init__(self, parent: HybridCache, b0: int, b1: int):
        self.parent = parent
        self.b0, self.b1 = b0, b1
        self.batch_size = b1 - b0
        self.max_length = parent.max_length
        self.specs = parent.specs

    @property
    def device(self):
        return self.parent.device

    @property
    def index(self):
        return self.parent.index

    @property
    def index_t(self):
        return self.parent.index_t

    def layer(self, i: int):
        k, v = self.parent.layer(i)
        return k[self.b0:self.b1], v[self.b0:self.b1]

    def owns_kv(self, i: int) -> bool:
        return self.parent.owns_kv(i)

    def recurrent(self, i: int):
        s, c = self.parent.recurrent(i)
        return s[self.b0:self.b1], c[self.b0:self.b1]
