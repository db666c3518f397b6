"""Per-head static + circular KV cache and the plan -> cache-size rule.

Same surface as the reference's ``StaticCircularCache``
(MoA/attention/cache_utils.py:644-1180) and ``moa_config_to_cache_config``
(:1183-1298).  The bookkeeping tensors keep the reference's names, shapes and
int64 dtype so that callers written against the reference keep working; the
work of ``update`` -- the row scatter and the ring-pointer arithmetic that the
reference spreads over ~15 torch indexing ops per layer-step -- is one call
into libmoa_hip.so (moa_cache_append / moa_cache_prefill_insert).
"""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional, Tuple

import torch
from torch import Tensor

from moa_amd import _lib


class StaticCircularCache:
    """A cache that does not grow as tokens are generated.

    Per layer the keys and values are one tensor
    ``[batch_size, sum_h cache_size_h, head_dim]``: head ``h`` owns a contiguous
    run of ``cache_size_h`` rows, the first ``static_size_h`` of which keep the
    first tokens forever (the sinks) while the rest is a ring holding the most
    recent tokens.  ``update`` takes ``[batch_size, num_heads, seq_len, head_dim]``.

    Unlike the reference this class does not derive from
    ``transformers.Cache``: the installed transformers release changed that base
    class incompatibly, and nothing on the attention path uses it.
    """

    def __init__(
        self,
        cache_size: List[List[int]],
        batch_size: int = 1,
        head_dim: int = 128,
        static_size: Optional[List[List[int]]] = None,
        device: torch.device = "cpu",
        dtype: torch.dtype = None,
        update_cache_content: bool = True,
    ) -> None:
        self.dtype = dtype if dtype is not None else torch.float16
        self.device = device
        self.update_cache_content = update_cache_content
        self.batch_size = batch_size
        self.head_dim = head_dim

        self.num_layers = len(cache_size)
        self.num_head_for_each_layer = [len(c) for c in cache_size]
        if static_size is None:
            static_size = [[0] * len(c) for c in cache_size]
        assert len(static_size) == self.num_layers
        for layer_id in range(self.num_layers):
            assert len(static_size[layer_id]) == len(cache_size[layer_id])
            for c, s in zip(cache_size[layer_id], static_size[layer_id]):
                assert 0 <= s <= c, "static size must lie within the cache size"

        def i64(x):
            return torch.tensor(x, device=device, dtype=torch.int64)

        self.cache_max_length: List[Tensor] = [i64(c) for c in cache_size]
        self.static_cache_size: List[Tensor] = [i64(s) for s in static_size]
        self.circular_cache_size: List[Tensor] = [
            c - s for c, s in zip(self.cache_max_length, self.static_cache_size)]
        self.layer_cache_size: List[int] = [sum(c) for c in cache_size]
        self._max_cache_size: List[int] = [max(c) for c in cache_size]
        self._max_static_size: List[int] = [max(x) for x in static_size]

        starts = []
        for c in cache_size:
            acc, row = 0, []
            for x in c:
                row.append(acc)
                acc += x
            starts.append(row)
        self.cache_head_start_index: List[Tensor] = [
            i64(starts[l])[None, :].expand(batch_size, -1).contiguous() for l in range(self.num_layers)]
        self.head_index: List[Tensor] = [
            i64(starts[l] + [starts[l][-1] + cache_size[l][-1]]) for l in range(self.num_layers)]
        self.circular_cache_head_index: List[Tensor] = [
            i64([a + s for a, s in zip(starts[l], static_size[l])]) for l in range(self.num_layers)]
        # materialised [B, H]: the append kernel advances it in place
        self.cache_update_index: List[Tensor] = [
            i64(starts[l])[None, :].expand(batch_size, -1).contiguous() for l in range(self.num_layers)]

        self.cache_position = 0
        self._kv_len = [0 for _ in range(self.num_layers)]
        self._ready_on: List[Optional[torch.device]] = [None] * self.num_layers   # device the layer's tensors are on
        self._step_args: List[Optional[Dict[str, Any]]] = [None] * self.num_layers   # what rope_update keeps per layer
        self._capturing: Optional[bool] = None   # is the stream capturing (asked once per step)

        # K/V are created on the device of the first update of each layer
        self.key_cache: List[Optional[Tensor]] = [None] * self.num_layers
        self.value_cache: List[Optional[Tensor]] = [None] * self.num_layers
        self.mask_cache: List[Tensor] = [
            torch.zeros(batch_size, n, dtype=torch.int64, device=device) for n in self.layer_cache_size]
        self.cache_valid_length: List[Tensor] = [
            torch.zeros((batch_size, h), dtype=torch.int64, device=device)
            for h in self.num_head_for_each_layer]

    def __getstate__(self):
        """Copies (copy.deepcopy, pickling) do not take the per-layer call arguments along: those hold
        device addresses of THIS object's tensors."""
        state = self.__dict__.copy()
        state["_step_args"] = [None] * self.num_layers
        return state

    # ------------------------------------------------------------------
    # layout helpers (same results as the reference's static methods)
    # ------------------------------------------------------------------
    @staticmethod
    def head_start_index_valid_length_to_head_index(head_start_index: Tensor,
                                                    head_valid_length: Tensor) -> Tensor:
        """MoA/attention/cache_utils.py:820-840."""
        assert (head_start_index == head_start_index[0]).all().item()
        assert (head_valid_length == head_valid_length[0]).all().item()
        head_index = torch.cat(
            (head_start_index[0], (head_start_index[0][-1] + head_valid_length[0][-1]).reshape(-1)))
        return head_index.contiguous()

    @staticmethod
    def head_index_to_head_start_index_valid_length(head_index: Tensor, batch_size: int = 1):
        """Raises, as in the reference (:842-851): a valid length cannot be
        recovered from segment boundaries."""
        raise NotImplementedError

    @staticmethod
    def to_uncontigious(tensor: Tensor, head_index: Tensor) -> List[Tensor]:
        """One ``[batch, cache_size_h, (head_dim)]`` slice per head (:867-887)."""
        return [tensor[:, head_index[h]:head_index[h + 1]] for h in range(len(head_index) - 1)]

    @staticmethod
    def to_group_contigious(tensor: Tensor, head_index: Tensor) -> List[Tensor]:
        """Runs of consecutive heads with equal cache size, each viewed
        ``[batch, heads_in_group, cache_size, (head_dim)]`` (:889-951)."""
        sizes = (head_index[1:] - head_index[:-1]).tolist()
        bounds = head_index.tolist()
        groups = []
        i, H = 0, len(sizes)
        while i < H:
            j = i
            while j + 1 < H and sizes[j + 1] == sizes[i]:
                j += 1
            count = j - i + 1
            sl = tensor[:, bounds[i]:bounds[j] + sizes[i]]
            shape = (tensor.shape[0], count, sizes[i]) + tuple(tensor.shape[2:])
            groups.append(sl.reshape(shape).contiguous())
            i = j + 1
        return groups

    # ------------------------------------------------------------------
    def _to_device(self, layer_idx: int, device: torch.device) -> None:
        if self._ready_on[layer_idx] == device:
            return
        for name in ("mask_cache", "cache_update_index", "cache_head_start_index",
                     "circular_cache_head_index", "cache_valid_length", "cache_max_length",
                     "circular_cache_size", "static_cache_size", "head_index"):
            lst = getattr(self, name)
            if lst[layer_idx].device != device:
                lst[layer_idx] = lst[layer_idx].to(device=device)
        if self.update_cache_content and self.key_cache[layer_idx] is None:
            shape = (self.batch_size, self.layer_cache_size[layer_idx], self.head_dim)
            self.key_cache[layer_idx] = torch.zeros(shape, dtype=self.dtype, device=device)
            self.value_cache[layer_idx] = torch.zeros(shape, dtype=self.dtype, device=device)
        self._ready_on[layer_idx] = device
        self._step_args[layer_idx] = None

    def _check_capture(self, layer_idx: int, device) -> None:
        """A decode step recorded into a HIP graph bakes in the host value ``kv_len``, which the
        append kernels use for one decision only: has this head left its static part (the reference's
        ``kv_len + 1 > static_size``, cache_utils.py:1041-1045).  A replay is right as long as that
        decision does not change any more, i.e. once every head of the layer is past its sinks.
        Capturing earlier would let replays walk a head's pointer linearly out of its segment.
        (Replays do not advance ``get_seq_length()`` / ``cache_position`` either: callers that replay
        pass explicit positions.)  Called before anything is changed, so a caller that catches the error
        can go on eagerly.  The stream is asked once per step (layer 0); the other layers of the step
        use that answer."""
        if layer_idx == 0 or self._capturing is None:
            self._capturing = torch.cuda.is_current_stream_capturing()
        if self._capturing and self._kv_len[layer_idx] + 1 <= self._max_static_size[layer_idx]:
            raise RuntimeError(
                f"StaticCircularCache: layer {layer_idx} has seen {self._kv_len[layer_idx]} tokens, not more than its "
                f"largest static size {self._max_static_size[layer_idx]}: a decode step captured now would be "
                "replayed with the wrong ring decision; capture after the prompt has filled the static parts")

    def rope_update(
        self,
        query_states: Tensor,
        key_states: Tensor,
        value_states: Tensor,
        cos: Tensor,
        sin: Tensor,
        layer_idx: int,
        attention_mask: Optional[torch.IntTensor] = None,
    ) -> Tuple[Tensor, Tensor, Tensor]:
        """Rotary embedding of q and k followed by ``update``: the two steps the reference's caller
        runs between the projections and the attention call (modeling_llama.py:252 and :262).

        q ``[batch, q_heads, seq_len, head_dim]``, k/v ``[batch, heads, seq_len, head_dim]`` before
        rotation, cos/sin ``[batch or 1, seq_len, head_dim]``.  Returns ``(q_embed, keys, values)``
        where keys/values are what ``update`` returns.  With ``seq_len == 1`` this is ONE launch:
        q is rotated into a ``[batch, 1, q_heads, head_dim]`` buffer (returned as its
        ``[batch, q_heads, 1, head_dim]`` view, the layout the decode kernel takes without a copy), k is
        rotated straight into its ring slot, v is copied into its slot.  That buffer belongs to the
        cache, one per layer, and is written again by the layer's next step.
        """
        from ..kernels.rotary import apply_rotary_pos_emb, _cos_sin_strides

        seq_len = key_states.shape[-2]
        if seq_len != 1 or not self.update_cache_content:
            q_embed, k_embed = apply_rotary_pos_emb(query_states, key_states, cos, sin)
            keys, values = self.update(k_embed, value_states, layer_idx, attention_mask)
            return q_embed, keys, values

        assert layer_idx < self.num_layers
        H = self.num_head_for_each_layer[layer_idx]
        device = key_states.device
        if device.type != "cuda":
            raise _lib.MoaKernelError(
                "StaticCircularCache.rope_update: tensors must live on the GPU; moa_amd has no CPU path")
        B, Hq, _, D = query_states.shape
        assert key_states.shape == (B, H, 1, D) and value_states.shape == key_states.shape
        assert B == self.batch_size and D == self.head_dim
        assert query_states.dtype == self.dtype and key_states.dtype == self.dtype and value_states.dtype == self.dtype
        assert cos.dtype == self.dtype and sin.dtype == self.dtype, "cos/sin must have the cache dtype"
        self._to_device(layer_idx, device)
        self._check_capture(layer_idx, device)

        # What does not change from step to step is kept per layer: the library handle, the pointers of the
        # cache and its index tensors, the q buffer, and the stride arrays of the last operand layout seen.
        st = self._step_args[layer_idx]
        layout = (query_states.stride(), key_states.stride(), value_states.stride(), cos.shape, cos.stride(),
                  sin.stride(), Hq)
        if st is None or st["layout"] != layout:
            qs, ks_, vs_ = query_states.stride(), key_states.stride(), value_states.stride()
            if qs[-1] != 1 or ks_[-1] != 1 or vs_[-1] != 1:
                st = None   # rare: operands without a contiguous head_dim are copied, nothing is kept
            else:
                upd = self.cache_update_index[layer_idx]
                assert upd.is_contiguous() and self.cache_valid_length[layer_idx].is_contiguous()
                _, _, css = _cos_sin_strides(cos, sin, B, 1, D)
                q_out = torch.empty((B, 1, Hq, D), dtype=self.dtype, device=device)
                st = {
                    "layout": layout, "lib": _lib.load(), "q_out": q_out, "q_view": q_out.transpose(1, 2),
                    "cos_ok": cos.stride(-1) == 1 and sin.stride() == cos.stride(),
                    "strides": (_lib.i64_array((qs[0], qs[1], qs[3])), _lib.i64_array((ks_[0], ks_[1], ks_[3])),
                                _lib.i64_array((vs_[0], vs_[1], vs_[3])), css[0]),
                    "tail": (q_out.data_ptr(), self.key_cache[layer_idx].data_ptr(),
                             self.value_cache[layer_idx].data_ptr(), self.mask_cache[layer_idx].data_ptr(),
                             upd.data_ptr(), self.cache_valid_length[layer_idx].data_ptr(),
                             self.circular_cache_head_index[layer_idx].data_ptr(),
                             self.circular_cache_size[layer_idx].data_ptr(),
                             self.static_cache_size[layer_idx].data_ptr(),
                             self.cache_max_length[layer_idx].data_ptr()),
                    "sizes": (B, Hq, H, D, self.layer_cache_size[layer_idx], _lib.dtype_code(self.dtype)),
                }
                self._step_args[layer_idx] = st
        if st is not None and st["cos_ok"]:
            qstr, kstr, vstr, cos_b = st["strides"]
            rc = st["lib"].moa_rope_cache_append(
                query_states.data_ptr(), key_states.data_ptr(), value_states.data_ptr(), qstr, kstr, vstr,
                cos.data_ptr(), sin.data_ptr(), cos_b, *st["tail"], self._kv_len[layer_idx], *st["sizes"],
                _lib.current_stream_ptr(device))
            q_view = st["q_view"]
        else:
            cos, sin, css = _cos_sin_strides(cos, sin, B, 1, D)
            qn, kn, vn = (t[:, :, -1, :] for t in (query_states, key_states, value_states))
            qn, kn, vn = (t if t.stride(-1) == 1 else t.contiguous() for t in (qn, kn, vn))
            q_out = torch.empty((B, 1, Hq, D), dtype=self.dtype, device=device)
            rc = _lib.load().moa_rope_cache_append(
                qn.data_ptr(), kn.data_ptr(), vn.data_ptr(), _lib.i64_array(qn.stride()), _lib.i64_array(kn.stride()),
                _lib.i64_array(vn.stride()), cos.data_ptr(), sin.data_ptr(), css[0], q_out.data_ptr(),
                self.key_cache[layer_idx].data_ptr(), self.value_cache[layer_idx].data_ptr(),
                self.mask_cache[layer_idx].data_ptr(), self.cache_update_index[layer_idx].data_ptr(),
                self.cache_valid_length[layer_idx].data_ptr(),
                self.circular_cache_head_index[layer_idx].data_ptr(),
                self.circular_cache_size[layer_idx].data_ptr(),
                self.static_cache_size[layer_idx].data_ptr(),
                self.cache_max_length[layer_idx].data_ptr(),
                self._kv_len[layer_idx], B, Hq, H, D, self.layer_cache_size[layer_idx],
                _lib.dtype_code(self.dtype), _lib.current_stream_ptr(device))
            q_view = q_out.transpose(1, 2)
        _lib.check(rc)
        if layer_idx == 0:
            self.cache_position += 1
        self._kv_len[layer_idx] += 1
        return q_view, self.key_cache[layer_idx], self.value_cache[layer_idx]

    def update(
        self,
        key_states: Tensor,
        value_states: Tensor,
        layer_idx: int,
        attention_mask: Optional[torch.IntTensor] = None,
        cache_kwargs: Optional[Dict[str, Any]] = None,
    ) -> Tuple[Tensor, Tensor]:
        """Stores new keys/values ``[batch, heads, seq_len, head_dim]``.

        ``seq_len == 1`` appends one token to every head's ring and returns the
        whole packed caches ``[batch, sum_h cache_size_h, head_dim]``
        (reference :1020-1058).  ``seq_len > 1`` inserts a prompt -- the first
        ``static`` tokens and the last ``circular`` ones survive -- and returns
        the inputs (:1060-1164).  ``attention_mask`` ``[batch, kv_len]`` int64
        of 0/1 marks padding in the prompt.
        """
        assert layer_idx < self.num_layers
        H = self.num_head_for_each_layer[layer_idx]
        if key_states is not None:
            assert key_states.shape[1] == H
            device = key_states.device
            assert value_states.device == device, "key_states and value_states should be on the same device"
        else:
            assert not self.update_cache_content, "key_states may be None only with update_cache_content=False"
            device = self.cache_update_index[layer_idx].device
        if attention_mask is not None:
            assert attention_mask.device == device, "attention_mask should be on the same device as key_states"
        if torch.device(device).type != "cuda":
            raise _lib.MoaKernelError(
                "StaticCircularCache.update: tensors must live on the GPU; moa_amd has no CPU path")
        lib = _lib.load()
        self._to_device(layer_idx, device)

        if self.update_cache_content:
            batch_size, seq_len, head_dim = key_states.shape[0], key_states.shape[-2], key_states.shape[-1]
            assert batch_size == self.batch_size and head_dim == self.head_dim
            assert key_states.dtype == self.dtype and value_states.dtype == self.dtype
            assert value_states.shape == key_states.shape
        else:
            batch_size = self.batch_size
            seq_len = key_states.shape[-2] if key_states is not None else 1
            head_dim = self.head_dim
        if seq_len == 1:
            self._check_capture(layer_idx, device)   # before anything is changed
        if layer_idx == 0:
            self.cache_position += seq_len

        sumC = self.layer_cache_size[layer_idx]
        stream = _lib.current_stream_ptr(device)
        dt = _lib.dtype_code(self.dtype)
        kc = self.key_cache[layer_idx] if self.update_cache_content else None
        vc = self.value_cache[layer_idx] if self.update_cache_content else None
        upd = self.cache_update_index[layer_idx]
        assert upd.is_contiguous() and self.cache_valid_length[layer_idx].is_contiguous()

        if seq_len == 1:
            kn = vn = None
            kns = vns = None
            if self.update_cache_content:
                kn = key_states[:, :, -1, :]
                vn = value_states[:, :, -1, :]
                if kn.stride(-1) != 1:
                    kn = kn.contiguous()
                if vn.stride(-1) != 1:
                    vn = vn.contiguous()
                kns = _lib.i64_array(kn.stride())
                vns = _lib.i64_array(vn.stride())
            rc = lib.moa_cache_append(
                _lib.ptr(kn), _lib.ptr(vn), kns, vns, _lib.ptr(kc), _lib.ptr(vc),
                self.mask_cache[layer_idx].data_ptr(), upd.data_ptr(),
                self.cache_valid_length[layer_idx].data_ptr(),
                self.circular_cache_head_index[layer_idx].data_ptr(),
                self.circular_cache_size[layer_idx].data_ptr(),
                self.static_cache_size[layer_idx].data_ptr(),
                self.cache_max_length[layer_idx].data_ptr(),
                self._kv_len[layer_idx], batch_size, H, head_dim, sumC, dt, stream)
            _lib.check(rc)
            self._kv_len[layer_idx] += 1
            return self.key_cache[layer_idx], self.value_cache[layer_idx]

        am_ptr, am_stride, ws_ptr, ws_bytes = None, 0, None, 0
        if attention_mask is not None:
            assert len(attention_mask.shape) == 2, (
                "The shape of the attention mask should be [batch_size, kv_len] and the dtype should be torch.int64.")
            am = attention_mask[:, -seq_len:]
            if am.dtype != torch.int64 or am.stride(-1) != 1:
                am = am.to(torch.int64).contiguous()
            am_ptr, am_stride = am.data_ptr(), am.stride(0)
            ws_bytes = lib.moa_cache_prefill_workspace_bytes(batch_size, seq_len)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
            ws_ptr = ws.data_ptr()
        ks = vs = None
        k_in, v_in = key_states, value_states
        if self.update_cache_content:
            if k_in.stride(-1) != 1:
                k_in = k_in.contiguous()
            if v_in.stride(-1) != 1:
                v_in = v_in.contiguous()
            ks = _lib.i64_array(k_in.stride())
            vs = _lib.i64_array(v_in.stride())
        rc = lib.moa_cache_prefill_insert(
            _lib.ptr(k_in) if self.update_cache_content else None,
            _lib.ptr(v_in) if self.update_cache_content else None, ks, vs,
            _lib.ptr(kc), _lib.ptr(vc), self.mask_cache[layer_idx].data_ptr(), upd.data_ptr(),
            self.cache_valid_length[layer_idx].data_ptr(),
            self.circular_cache_head_index[layer_idx].data_ptr(),
            self.circular_cache_size[layer_idx].data_ptr(),
            self.static_cache_size[layer_idx].data_ptr(),
            am_ptr, am_stride, ws_ptr, ws_bytes, self._kv_len[layer_idx], batch_size, H, seq_len,
            head_dim, sumC, self._max_cache_size[layer_idx], dt, stream)
        _lib.check(rc)
        self._kv_len[layer_idx] += seq_len
        return key_states, value_states

    def __len__(self):
        return self.num_layers

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        """Number of token positions this layer has been shown (padding included)."""
        return self._kv_len[layer_idx]

    def get_max_length(self) -> Optional[int]:
        return None

    def reorder_cache(self, beam_idx: torch.LongTensor):
        raise NotImplementedError("Reordering the cache is not implemented currently!")


def moa_config_to_cache_config(
    moa_config,
    seq_len,
    max_new_token: int = 1024,
    sink_size: int = 64,
    minimum_cache_size: int = 128,
    split_size: int = 64,
    verbose: bool = True,
):
    """Plan ``{"alphas": [L][H], "betas": [L][H]}`` -> per-head cache sizes.

    Rule of the reference (MoA/attention/cache_utils.py:1224-1237), evaluated once at
    ``N = seq_len + max_new_token``:
        cache = ceil(max(min(int(alpha + N * beta), N), minimum_cache_size) / split_size) * split_size
        static = min(cache, sink_size)
    Returns ``{"cache_size": [L][H], "static_size": [L][H]}``.
    """
    alphas, betas = moa_config["alphas"], moa_config["betas"]
    n_total = seq_len + max_new_token
    cache_size, static_size = [], []
    for layer_alphas, layer_betas in zip(alphas, betas):
        cs, ss = [], []
        for a, b in zip(layer_alphas, layer_betas):
            c = min(int(a + n_total * b), n_total)
            c = math.ceil(max(c, minimum_cache_size) / split_size) * split_size
            cs.append(c)
            ss.append(min(c, sink_size))
        cache_size.append(cs)
        static_size.append(ss)
    if verbose:
        print("Cache configuration")
        print(format_cache_summary(*cache_config_summary(cache_size, static_size, n_total)))
    return {"cache_size": cache_size, "static_size": static_size}


_SUMMARY_METRICS = ("cache_size", "static_size", "circular_size", "ratio")


def cache_config_summary(cache_size, static_size, raw_cache_size):
    """What the reference prints for a cache configuration (MoA/attention/cache_utils.py:1241-1293), as
    data: per layer the mean raw size (``seq_len + max_new_token``) and the (mean, min, max) over heads
    of cache_size, static_size, circular_size = cache - static and ratio = cache / raw; for the whole
    model the same four metrics plus raw_cache_size over all heads.  Returns ``(layer_rows, model_rows)``:
    ``layer_rows[l][metric] = (mean, min, max)`` and ``model_rows[metric] = (mean, min, max)``."""
    def stats(xs):
        return (sum(xs) / len(xs), min(xs), max(xs))

    def metrics(cs, ss):
        return {"cache_size": list(cs), "static_size": list(ss), "circular_size": [c - s for c, s in zip(cs, ss)],
                "ratio": [c / raw_cache_size for c in cs]}

    layer_rows = []
    for cs, ss in zip(cache_size, static_size):
        row = {k: stats(v) for k, v in metrics(cs, ss).items()}
        row["raw_cache_size"] = (float(raw_cache_size),) * 3
        layer_rows.append(row)
    flat_c = [c for cs in cache_size for c in cs]
    flat_s = [x for ss in static_size for x in ss]
    model_rows = {k: stats(v) for k, v in metrics(flat_c, flat_s).items()}
    model_rows["raw_cache_size"] = (float(raw_cache_size),) * 3
    return layer_rows, model_rows


def format_cache_summary(layer_rows, model_rows) -> str:
    """The two tables of the reference's printout (per layer, then the model), two decimals like its
    ``pd.options.display.float_format``; plain text, no pandas."""
    head = f"{'layer_id':>8} {'raw_cache_size':>14}" + "".join(
        f" {m + ' mean':>19} {'min':>9} {'max':>9}" for m in _SUMMARY_METRICS)
    lines = [head]
    for l, row in enumerate(layer_rows):
        line = f"{l:>8} {row['raw_cache_size'][0]:>14.2f}"
        for m in _SUMMARY_METRICS:
            mean, lo, hi = row[m]
            line += f" {mean:>19.2f} {lo:>9.2f} {hi:>9.2f}"
        lines.append(line)
    lines.append(f"{'metric':>16} {'max':>12} {'mean':>12} {'min':>12}")
    for m in ("cache_size", "circular_size", "ratio", "raw_cache_size", "static_size"):
        mean, lo, hi = model_rows[m]
        lines.append(f"{m:>16} {hi:>12.2f} {mean:>12.2f} {lo:>12.2f}")
    return "\n".join(lines)
