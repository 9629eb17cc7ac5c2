"""
Streaming KV cache over the TurboQuant V3 codec.

`V3Cache.update(key_states, value_states, layer_idx)` has the contract of the reference's
generation-time cache (turboquant/generation_test_v2.py:48-165): new tokens join an uncompressed
window of the most recent `residual_window` tokens, tokens pushed out of the window are
compressed for good, and every call returns the full-length keys and values of the layer --
de-quantised old tokens followed by the window -- in the dtype of the incoming states.

What is different underneath:
  * the reference keeps a Python list of compressed chunks per layer and de-quantises them one
    by one on every step (O(steps) small launches, then a concatenation).  Here each layer owns
    one preallocated packed store [B, H, capacity, G] (+ fp16 norms); tokens leaving the window are
    appended in place (`packed_row_stride` of the C ABI), and a step is one compress launch per
    tensor for the leaving tokens plus one decompress launch per tensor that writes the whole
    history straight into the output buffer;
  * codes depend on the vector alone, so the stored bytes are the same whatever the chunking.
The class does not derive from transformers' DynamicCache; `hf_cache_class()` builds that
subclass when transformers is importable.
"""
from __future__ import annotations

from typing import Dict, NamedTuple, Optional, Tuple

import torch

from . import _native
from .compressors_v3 import TurboQuantV3


class _StepConsts(NamedTuple):
    """What the per-token library calls of one layer pass on every step: device addresses and sizes."""
    k_win: int
    v_win: int
    win_stride: int        # elements between rows of the window buffers
    table_k: int
    table_v: int
    bits_k: int
    bits_v: int
    k_idx: int
    k_nrm: int
    v_idx: int
    v_nrm: int
    pi_k_t: int
    pi_v: int
    dtype: int
    vec_bytes: int         # bytes of one window token


class _LayerStore:
    """Packed history and uncompressed window of one layer."""

    def __init__(self, comp: TurboQuantV3, B: int, H: int, D: int, dtype: torch.dtype, device: torch.device,
                 capacity: int, window: int):
        self.comp = comp
        self.B, self.H, self.D = B, H, D
        self.dtype, self.device = dtype, device
        self.capacity = 0
        self.k_idx = self.k_nrm = self.v_idx = self.v_nrm = None
        self.n_compressed = 0
        self.window_tokens = window
        # the window store holds the uncompressed tail between calls: tokens [w0, w0 + n_recent) of a
        # buffer twice the window long, so that it is moved back to the front once per `window` steps
        # (+8 tokens: rows of the buffer then do not start a power of two apart, see reserve)
        self.win_cap = max(2 * window + 8, 1)
        self.k_win = torch.empty((B, H, self.win_cap, D), dtype=dtype, device=device)
        self.v_win = torch.empty_like(self.k_win)
        self.w0 = 0
        self.n_recent = 0
        self.total_seq = 0
        self._consts = None
        self.reserve(capacity)

    @staticmethod
    def _width(D: int, bits: int) -> int:
        ipb = 8 // bits
        return -(-D // ipb)

    def reserve(self, tokens: int) -> None:
        """Make room for `tokens` compressed tokens per (batch, head) row (amortised doubling)."""
        if tokens <= self.capacity:
            return
        cap = max(tokens, 2 * self.capacity, 256)
        cap = -(-cap // 64) * 64
        if cap % 1024 == 0:
            # Rows a large power of two apart start on the same memory channels, and the kernels that walk all
            # rows at the same pace then queue up on them: 238 instead of 195 us for the attention pass over
            # 512 rows x 16384 tokens.
            cap += 64
        new = []
        for old, width in ((self.k_idx, self._width(self.D, self.comp.key_bits)), (self.k_nrm, None),
                           (self.v_idx, self._width(self.D, self.comp.value_bits)), (self.v_nrm, None)):
            if width is None:
                buf = torch.empty((self.B, self.H, cap), dtype=torch.float16, device=self.device)
            else:
                buf = torch.empty((self.B, self.H, cap, width), dtype=torch.uint8, device=self.device)
            if old is not None and self.n_compressed:
                buf[:, :, :self.n_compressed].copy_(old[:, :, :self.n_compressed])
            new.append(buf)
        self.k_idx, self.k_nrm, self.v_idx, self.v_nrm = new
        self.capacity = cap
        self._consts = None

    def consts(self) -> _StepConsts:
        """Rebuilt when the packed store moves (`reserve`)."""
        c = self._consts
        if c is None:
            kc, vc = self.comp.key_compressor, self.comp.val_compressor
            c = self._consts = _StepConsts(
                self.k_win.data_ptr(), self.v_win.data_ptr(), self.win_cap * self.D,
                kc.table().data_ptr(), vc.table().data_ptr(), kc.bits, vc.bits,
                self.k_idx.data_ptr(), self.k_nrm.data_ptr(), self.v_idx.data_ptr(), self.v_nrm.data_ptr(),
                kc.pi_transposed().data_ptr(), vc.Pi.data_ptr(), _native.dtype_code(self.dtype),
                self.D * self.k_win.element_size())
        return c

    def append_one(self, keys: torch.Tensor, values: torch.Tensor) -> bool:
        """The steady-state decode step in one library call: the window is full, its oldest token is compressed
        into the next packed slot and the new token takes the next window slot.  False (nothing done) when the
        step is not of that kind or the tensors are not laid out for it; the general path then runs."""
        rw = self.window_tokens
        if (rw == 0 or self.D != _native.HEAD_DIM      # (the one-call step exists for the 128-wide kernels only)
                or self.n_recent != rw or self.w0 + rw + 1 > self.win_cap or self.n_compressed + 1 > self.capacity
                or keys.dtype != self.dtype or values.dtype != self.dtype or keys.device != self.device
                or values.device != self.device or torch.compiler.is_compiling()):
            return False
        rows = self.B * self.H
        strides = []
        for t in (keys, values):
            s0, s1, _, s3 = t.stride()
            if s3 != 1 or (self.B > 1 and self.H > 1 and s0 != self.H * s1):
                return False
            strides.append(s1 if self.H > 1 else s0)
        if rows > 1 and min(strides) < self.D:           # broadcast views: the general path copies them
            return False
        c = self.consts()
        dev = self.device
        with _native._on(dev):
            rc = _native.lib().tq_append_token(keys.data_ptr(), values.data_ptr(), c.dtype, strides[0], strides[1],
                                               c.k_win, c.v_win, c.win_stride, self.w0, self.w0 + rw,
                                               c.table_k, c.table_v, self.D, c.bits_k, c.bits_v,
                                               c.k_idx, c.k_nrm, c.v_idx, c.v_nrm, self.capacity, self.n_compressed, rows,
                                               _native._stream_handle(dev))
        if rc == _native.ERR_ALIGN:
            return False
        _native.check(rc, "tq_append_token")
        self.n_compressed += 1
        self.w0 += 1
        self.total_seq += 1
        return True

    def append_compressed(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        """Compress [B,H,n,D] views of keys / values into packed slots [n_compressed, n_compressed + n)."""
        n = keys.shape[2]
        if n == 0:
            return
        self.reserve(self.n_compressed + n)
        lo, hi = self.n_compressed, self.n_compressed + n
        kc, vc = self.comp.key_compressor, self.comp.val_compressor
        kc.compress_into(keys, self.k_idx[:, :, lo:hi], self.k_nrm[:, :, lo:hi])
        vc.compress_into(values, self.v_idx[:, :, lo:hi], self.v_nrm[:, :, lo:hi])
        self.n_compressed = hi

    def window(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Views [B,H,n_recent,D] of the uncompressed keys and values, oldest first."""
        return (self.k_win[:, :, self.w0:self.w0 + self.n_recent], self.v_win[:, :, self.w0:self.w0 + self.n_recent])

    def extend_window(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        n = keys.shape[2]
        if n == 0:
            return
        if self.w0 + self.n_recent + n > self.win_cap:
            if self.n_recent:
                k, v = self.window()
                k, v = k.clone(), v.clone()
                self.k_win[:, :, :self.n_recent].copy_(k)
                self.v_win[:, :, :self.n_recent].copy_(v)
            self.w0 = 0
        lo = self.w0 + self.n_recent
        self.k_win[:, :, lo:lo + n].copy_(keys)
        self.v_win[:, :, lo:lo + n].copy_(values)
        self.n_recent += n


class V3Cache:
    """Streaming compressed KV cache; `update` follows generation_test_v2.py:80-153."""

    def __init__(self, key_bits: int = 4, value_bits: int = 2, residual_window: int = 128,
                 protected_layers: int = 0, n_layers: int = 36, *, capacity: int = 0):
        self.key_bits = key_bits
        self.value_bits = value_bits
        self.residual_window = residual_window
        self.protected_layers = protected_layers
        self.n_layers = n_layers
        self.capacity = capacity          # expected compressed tokens per sequence (0: grow on demand)
        self._compressors: Dict[int, TurboQuantV3] = {}
        self._stores: Dict[int, _LayerStore] = {}

    def _get_compressor(self, layer_idx: int, head_dim: int, device) -> TurboQuantV3:
        # generation_test_v2.py:65-78: per-layer codec, residual_window=0 (the cache owns the window)
        if layer_idx not in self._compressors:
            self._compressors[layer_idx] = TurboQuantV3(
                head_dim=head_dim,
                key_bits=self.key_bits,
                value_bits=self.value_bits,
                residual_window=0,
                layer_idx=layer_idx,
                n_layers=self.n_layers,
                protected_layers=self.protected_layers,
                seed=42,
                device=str(device),
            )
        return self._compressors[layer_idx]

    def _store(self, key_states: torch.Tensor, layer_idx: int) -> _LayerStore:
        B, H, _, D = key_states.shape
        device = key_states.device
        comp = self._get_compressor(layer_idx, D, device)
        st = self._stores.get(layer_idx)
        if st is None:
            st = _LayerStore(comp, B, H, D, key_states.dtype, device, self.capacity, self.residual_window)
            self._stores[layer_idx] = st
        elif (st.B, st.H, st.D) != (B, H, D):
            raise ValueError(f"layer {layer_idx}: states {tuple(key_states.shape)} do not match the cached "
                             f"batch/head/dim {(st.B, st.H, st.D)}")
        return st

    def _push(self, st: _LayerStore, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        """Bookkeeping of generation_test_v2.py:96-126: the uncompressed tokens are (window ++ new); all but
        the last `residual_window` of them are compressed for good, the rest is the new window."""
        S_new = key_states.shape[2]
        if S_new == 1 and st.append_one(key_states, value_states):
            return
        st.total_seq += S_new
        rw = self.residual_window
        recent = st.n_recent + S_new
        overflow = recent if rw == 0 else max(recent - rw, 0)
        from_window = min(overflow, st.n_recent)
        from_new = overflow - from_window
        kw, vw = st.window()
        st.append_compressed(kw[:, :, :from_window], vw[:, :, :from_window])
        st.append_compressed(key_states[:, :, :from_new], value_states[:, :, :from_new])
        st.w0 += from_window
        st.n_recent -= from_window
        if st.n_recent == 0:
            st.w0 = 0
        st.extend_window(key_states[:, :, from_new:], value_states[:, :, from_new:])

    @torch.no_grad()
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        B, H, S_new, D = key_states.shape
        device = key_states.device
        st = self._store(key_states, layer_idx)
        comp = st.comp
        self._push(st, key_states, value_states)
        n_c = st.n_compressed
        total = n_c + st.n_recent
        full_k = torch.empty((B, H, total, D), dtype=key_states.dtype, device=device)
        full_v = torch.empty((B, H, total, D), dtype=value_states.dtype, device=device)
        if n_c:
            comp.key_compressor.decompress_packed(st.k_idx[:, :, :n_c], st.k_nrm[:, :, :n_c], full_k[:, :, :n_c])
            comp.val_compressor.decompress_packed(st.v_idx[:, :, :n_c], st.v_nrm[:, :, :n_c], full_v[:, :, :n_c])
        if st.n_recent:
            kw, vw = st.window()
            full_k[:, :, n_c:].copy_(kw)
            full_v[:, :, n_c:].copy_(vw)
        return full_k, full_v

    @torch.no_grad()
    def append(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int) -> None:
        """`update` without building the full-length tensors: the state afterwards is the same.  For decode
        loops that read the cache through `attend`."""
        self._push(self._store(key_states, layer_idx), key_states, value_states)

    @torch.no_grad()
    def attend(self, query_states: torch.Tensor, layer_idx: int, scale: Optional[float] = None,
               fused: Optional[bool] = None) -> torch.Tensor:
        """softmax(scale * q K^T) V of one query token per sequence, [B,Hq,1,D] -> [B,Hq,1,D], over everything
        cached for the layer -- what the model computes from the tensors `update` returns -- read
        straight from the packed store.  Query head j uses kv head j // (Hq / H).
        fused (default: whenever at most 16 query heads share a kv head): one kernel pass over packed keys and
        values with an online softmax per split of the history; otherwise three steps (scores from the packed
        keys, softmax in float32, weighted sum of the packed values).  Window tokens are used as they are."""
        st = self._stores.get(layer_idx)
        if st is None or st.total_seq == 0:
            raise ValueError(f"attend: nothing is cached for layer {layer_idx}")
        B, Hq, Sq, D = query_states.shape
        if Sq != 1 or B != st.B or Hq % st.H:
            raise ValueError(f"attend needs one query token per sequence, [B={st.B}, k*{st.H}, 1, {st.D}]; got {tuple(query_states.shape)}")
        G = Hq // st.H
        scale = D ** -0.5 if scale is None else scale
        n_c, n_w = st.n_compressed, st.n_recent
        kc, vc = st.comp.key_compressor, st.comp.val_compressor
        if D != _native.HEAD_DIM:
            # The kernels that read packed codes directly are built for 128-wide heads.  Other head dimensions: the history
            # is de-quantised by the codec kernels (into float32: rounding the keys to 16 bits would move logits of the size
            # this cache sees by several per cent of a softmax weight) and attended to together with the window.
            k = torch.empty((B, st.H, n_c + n_w, D), dtype=torch.float32, device=query_states.device)
            v = torch.empty_like(k)
            if n_c:
                kc.decompress_packed(st.k_idx[:, :, :n_c], st.k_nrm[:, :, :n_c], k[:, :, :n_c])
                vc.decompress_packed(st.v_idx[:, :, :n_c], st.v_nrm[:, :, :n_c], v[:, :, :n_c])
            if n_w:
                kw, vw = st.window()
                k[:, :, n_c:] = kw
                v[:, :, n_c:] = vw
            q5 = query_states.reshape(B, st.H, G, D).float()
            probs = torch.softmax(torch.matmul(q5, k.transpose(-2, -1)) * scale, dim=-1)
            return torch.matmul(probs, v).to(query_states.dtype).reshape(B, Hq, 1, D)
        if fused is None:
            fused = G <= 16
        if fused and n_w <= 512 and not torch.compiler.is_compiling():
            out = self._attend_step(st, query_states, G, float(scale))
            if out is not None:
                return out
        kw, vw = st.window()
        if fused and n_w <= 512:
            # three launches: rotate the queries + window statistics, one pass over the packed history,
            # log-sum-exp merge + rotation back + cast
            if n_c:
                packed = (st.k_idx[:, :, :n_c], st.k_nrm[:, :, :n_c], st.v_idx[:, :, :n_c], st.v_nrm[:, :, :n_c])
            else:                                   # nothing has left the window yet: an empty history
                dev = query_states.device
                packed = (torch.empty((B, st.H, 0, 1), dtype=torch.uint8, device=dev),
                          torch.empty((B, st.H, 0), dtype=torch.float16, device=dev)) * 2
            return _native.call("attend_packed", query_states, *packed, kc.table(), vc.table(),
                                                 kc.bits, vc.bits, kc.pi_transposed(), vc.Pi, kw, vw, float(scale))
        # rows padded to a multiple of 8 floats (the kernels read weights with 16-byte loads); the padding
        # scores are -inf, so the softmax runs over the whole contiguous buffer
        q4 = query_states.reshape(B, st.H, G, D).to(torch.float32)
        total = n_c + n_w
        width = -(-total // 8) * 8
        scores = torch.empty((B, Hq, width), dtype=torch.float32, device=query_states.device)
        if width > total:
            scores[:, :, total:] = float("-inf")
        if n_c:
            kc.packed_scores(st.k_idx[:, :, :n_c], st.k_nrm[:, :, :n_c], query_states, scale, out=scores[:, :, :n_c])
        if n_w:
            scores[:, :, n_c:total] = (torch.matmul(q4, kw.to(torch.float32).transpose(-2, -1)) * scale).reshape(B, Hq, n_w)
        probs = torch.softmax(scores, dim=-1)
        if n_c:
            out = vc.packed_weighted_values(st.v_idx[:, :, :n_c], st.v_nrm[:, :, :n_c], probs[:, :, :n_c])
        else:
            out = torch.zeros((B, Hq, D), dtype=torch.float32, device=query_states.device)
        if n_w:
            out = out + torch.matmul(probs[:, :, n_c:total].reshape(B, st.H, G, n_w), vw.to(torch.float32)).reshape(B, Hq, D)
        return out.to(query_states.dtype).reshape(B, Hq, 1, D)

    @staticmethod
    def _attend_step(st: _LayerStore, query_states: torch.Tensor, G: int, scale: float) -> Optional[torch.Tensor]:
        """The fused path of `attend` in one library call (rotate + window, packed history, merge), with the
        scratch kept per stream.  None when the queries are not laid out for it."""
        B, Hq, _, D = query_states.shape
        if (not query_states.is_contiguous() or query_states.dtype not in _native._DTYPE_CODE or st.k_idx is None
                or query_states.device != st.device):
            return None
        n_c, n_w = st.n_compressed, st.n_recent
        rows = B * st.H
        L = _native.lib()
        dev = st.device
        c = st.consts()
        splits = L.tq_attend_splits(rows, n_c) if n_c else 0
        rec = D + 2
        n_q, n_pw, n_p = rows * G * D, rows * G * rec, rows * splits * G * rec
        with _native._on(dev):
            stream = _native._stream_handle(dev)
            scratch = _native.step_scratch(dev, stream, n_q + n_pw + n_p)
            if scratch is None:
                return None
            base = scratch.data_ptr()
            out = torch.empty_like(query_states)
            code = _native.dtype_code(query_states.dtype)
            win_off = st.w0 * c.vec_bytes
            rc = L.tq_attend_step(query_states.data_ptr(), code, rows, G, scale, c.pi_k_t, c.pi_v,
                                  c.k_win + win_off, c.v_win + win_off, c.dtype, n_w, c.win_stride,
                                  c.k_idx, c.k_nrm, c.v_idx, c.v_nrm, st.capacity, n_c,
                                  c.table_k, c.table_v, D, c.bits_k, c.bits_v,
                                  base, base + 4 * n_q, base + 4 * (n_q + n_pw), splits, out.data_ptr(), code, stream)
        _native.check(rc, "tq_attend_step")
        return out

    def get_seq_length(self, layer_idx: int = 0) -> int:
        st = self._stores.get(layer_idx)
        return st.total_seq if st is not None else 0

    def get_compression_info(self) -> str:
        if not self._stores:
            return "no compression"
        st = self._stores.get(0)
        comp = st.n_compressed if st is not None else 0
        total = st.total_seq if st is not None else 0
        return f"{comp} compressed, {total - comp} fp16, {total} total"

    def save(self, path: str, include_codec: bool = True) -> None:
        """Write configuration, packed history and window of every layer to one safetensors file."""
        from .serialize import save_cache
        save_cache(self, path, include_codec=include_codec)

    @classmethod
    def load(cls, path: str, device="cuda") -> "V3Cache":
        """A cache in the state `save` wrote: `update` / `append` / `attend` continue from there."""
        from .serialize import load_cache
        return load_cache(path, device=device, cls=cls)

    def stored_bytes(self) -> int:
        """Bytes held for the tokens seen so far (packed codes, norms, window), over all layers."""
        n = 0
        for st in self._stores.values():
            rows = st.B * st.H
            if st.n_compressed:
                n += rows * st.n_compressed * (st.k_idx.shape[-1] + st.v_idx.shape[-1] + 4)
            n += 2 * rows * st.n_recent * st.D * st.k_win.element_size()
        return n


def hf_cache_class():
    """A `V3Cache` that also derives from transformers.DynamicCache, so that it can be passed as
    `past_key_values` to `model.generate` the way generation_test_v2.py:178-201 does.

    With `packed_attention=True` (keyword of the returned class) decode steps do not de-quantise the history:
    `update` only appends the new token and hands it back tagged, and the attention function registered by
    `register_packed_attention()` computes the step's attention straight from the packed store (`attend`).
    Prefill (more than one new token) takes the ordinary path.  Batches must not be padded in that mode: every
    cached token is attended to."""
    from transformers import DynamicCache

    class HFV3Cache(V3Cache, DynamicCache):
        def __init__(self, *args, packed_attention: bool = False, **kwargs):
            DynamicCache.__init__(self)
            V3Cache.__init__(self, *args, **kwargs)
            self.packed_attention = packed_attention
            # A packed decode step hands the model only the new token's K / V.  Until `packed_attention_forward` has
            # answered it from the packed store the step is "pending"; anything else that touches the cache first
            # means the model's attention ran over one token (another attention implementation is selected, or the
            # tag on the key tensor was lost on the way), and that must not pass silently.
            self._pending_layer = None
            self._mask_checked = None      # (address, version, shape, cache length) of the last attention mask found free of padding

        def _no_pending(self, what: str) -> None:
            if self._pending_layer is not None:
                layer, self._pending_layer = self._pending_layer, None
                raise RuntimeError(
                    f"packed_attention: the decode step appended to layer {layer} was never answered by "
                    f"packed_attention_forward (next cache call: {what}).  The model's attention ran over the new token "
                    "alone.  Select the registered implementation (register_packed_attention(), "
                    "model.config._attn_implementation = 'tq_packed') or create the cache with packed_attention=False.")

        def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
            self._no_pending(f"update(layer {layer_idx})")
            if self.packed_attention and key_states.shape[2] == 1 and V3Cache.get_seq_length(self, layer_idx) > 0:
                V3Cache.append(self, key_states, value_states, layer_idx)
                key_states._tq_packed = (self, layer_idx)       # read by packed_attention_forward
                self._pending_layer = layer_idx
                out = (key_states, value_states)
            else:
                out = V3Cache.update(self, key_states, value_states, layer_idx, cache_kwargs)
            layers = getattr(self, "layers", None)
            if layers is not None:
                from transformers.cache_utils import DynamicLayer
                while len(layers) <= layer_idx:
                    layers.append(DynamicLayer())
            return out

        def get_seq_length(self, layer_idx=0):
            self._no_pending("get_seq_length")
            return V3Cache.get_seq_length(self, layer_idx)

        def get_mask_sizes(self, query_length, layer_idx=0):
            # (length, offset) of the keys the next update() of this layer will return
            return V3Cache.get_seq_length(self, layer_idx) + int(query_length), 0

    return HFV3Cache


def _mask_hides_nothing(mask: torch.Tensor) -> bool:
    """True if an attention mask (boolean: True = attend; additive: 0 = attend) lets every key through."""
    if mask.dtype == torch.bool:
        return bool(mask.all())
    return bool((mask == 0).all())


def packed_attention_forward(module, query, key, value, attention_mask, scaling=None, dropout=0.0, **kwargs):
    """Attention function for transformers' AttentionInterface.  A decode step whose keys come tagged from a
    cache in packed-attention mode is answered by `V3Cache.attend` (scores, softmax and value sum computed from
    the packed codes).  `attend` counts every cached token, so a mask that hides one (a padded batch) is refused;
    the mask of a step is inspected once, not once per layer.  Everything else is passed to the library's
    scaled-dot-product implementation unchanged."""
    tag = getattr(key, "_tq_packed", None)
    if tag is not None and query.shape[2] == 1:
        cache, layer_idx = tag
        if attention_mask is not None:
            # One inspection per decode step: the key carries the cache length of this step, so that a new mask that the
            # allocator happens to place at the address of the last one (fixed-length masks) is looked at again.
            ident = (attention_mask.data_ptr(), attention_mask._version, tuple(attention_mask.shape),
                     V3Cache.get_seq_length(cache, layer_idx))
            if cache._mask_checked != ident:
                if torch.cuda.is_current_stream_capturing():
                    # the inspection reads a device value on the host, which a stream capture cannot record
                    raise RuntimeError("packed_attention: an attention mask cannot be inspected while a graph is being captured; "
                                       "capture decode steps without a mask (unpadded batches need none) or use packed_attention=False.")
                if not _mask_hides_nothing(attention_mask):
                    raise RuntimeError("packed_attention: the attention mask hides cached tokens (padded batch?); attention from "
                                       "the packed store counts every cached token.  Use packed_attention=False for such batches.")
                cache._mask_checked = ident
        out = cache.attend(query, layer_idx, scale=scaling)           # [B, Hq, 1, D]
        if cache._pending_layer == layer_idx:
            cache._pending_layer = None
        return out.transpose(1, 2).contiguous(), None
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    return ALL_ATTENTION_FUNCTIONS["sdpa"](module, query, key, value, attention_mask, dropout=dropout, scaling=scaling, **kwargs)


def register_packed_attention(name: str = "tq_packed") -> str:
    """Register `packed_attention_forward` under `name`; select it with
    `model.config._attn_implementation = name` (or `model.set_attn_implementation(name)`).
    The library's scaled-dot-product mask builder is registered under the same name: without one, transformers
    hands a custom attention function no mask at all, and a padded batch would be attended to in full with no way
    for the function to notice."""
    from transformers import AttentionInterface
    AttentionInterface.register(name, packed_attention_forward)
    try:
        from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
        AttentionMaskInterface.register(name, sdpa_mask)
    except ImportError:          # releases that build masks inside the model: they pass them to every attention function
        pass
    return name
