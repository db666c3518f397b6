"""The caller of the attention path: a Llama-shaped attention layer that runs on moa_amd's kernels.

Mirrors ``LlamaMixtureAttention.forward`` and ``LlamaModel.set_mixture_of_attention`` of the
reference (MoA/models/llama/modeling_llama.py:206-332 and :334-406) without depending on a
particular transformers version: the projections are ``torch.nn.Linear`` (rocBLAS/hipBLASLt GEMMs,
outside the accelerated path), everything between them goes through libmoa_hip.so:

    q, k, v projections -> rotary embedding + cache update (one launch in decode)
                        -> mixture_of_sparse_attention (sparse prefill / ring decode) -> o_proj

Unlike the reference (which asserts one key-value group, :220-224) grouped-query attention is
accepted: the cache and the sparsity plan are per kv head.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor, nn

from moa_amd.attention.cache_utils import StaticCircularCache, moa_config_to_cache_config
from moa_amd.attention.permutation_utils import (moa_config_to_permutation, permute_attention_projection,
                                                 permute_output_projection)
from moa_amd.kernels.mixture_of_attention import mixture_of_sparse_attention


def rotary_cos_sin(position_ids: Tensor, head_dim: int, dtype: torch.dtype, base: float = 10000.0
                   ) -> Tuple[Tensor, Tensor]:
    """cos/sin ``[batch, seq_len, head_dim]`` of the default Llama rotary embedding
    (inv_freq = base^(-2i/d) in fp32, emb = cat(freqs, freqs), cast to ``dtype``)."""
    dev = position_ids.device
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64, device=dev).float() / head_dim))
    freqs = position_ids.float()[:, :, None] * inv_freq[None, None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def attention_geometry(attn) -> Tuple[int, int, int]:
    """(query heads, kv heads, head_dim) of an attention module: this package's LlamaMixtureAttention or
    a transformers Llama attention (whose head counts live in its config)."""
    cfg = getattr(attn, "config", None)
    num_heads = getattr(attn, "num_heads", None) or cfg.num_attention_heads
    num_kv = getattr(attn, "num_key_value_heads", None) or getattr(cfg, "num_key_value_heads", None) or num_heads
    head_dim = getattr(attn, "head_dim", None) or attn.q_proj.out_features // num_heads
    return int(num_heads), int(num_kv), int(head_dim)


def mixture_attention_forward(attn, hidden_states: Tensor, position_embeddings: Tuple[Tensor, Tensor],
                              past_key_value: StaticCircularCache, attention_mask: Optional[Tensor] = None) -> Tensor:
    """The body of the reference's ``LlamaMixtureAttention.forward`` (modeling_llama.py:232-326) for any
    module ``attn`` with ``q_proj / k_proj / v_proj / o_proj`` and a ``layer_idx``: projections, rotary
    embedding + cache update (one launch in decode), sparse attention, output projection.
    hidden_states ``[batch, q_len, hidden]``; position_embeddings ``(cos, sin)`` each
    ``[batch or 1, q_len, head_dim]``; attention_mask ``[batch, kv_len]`` of 0/1 marks left padding of a
    prompt.  Returns ``[batch, q_len, hidden]``."""
    assert not attn.training, "only support inference now"
    assert isinstance(past_key_value, StaticCircularCache)
    num_heads, num_kv, head_dim = attention_geometry(attn)
    bsz, q_len, _ = hidden_states.shape
    # [B, q_len, H*D] viewed as [B, H, q_len, D]: no copy, the kernels take the strides
    q = attn.q_proj(hidden_states).view(bsz, q_len, num_heads, head_dim).transpose(1, 2)
    k = attn.k_proj(hidden_states).view(bsz, q_len, num_kv, head_dim).transpose(1, 2)
    v = attn.v_proj(hidden_states).view(bsz, q_len, num_kv, head_dim).transpose(1, 2)
    cos, sin = position_embeddings
    li = attn.layer_idx
    q, keys, values = past_key_value.rope_update(q, k, v, cos, sin, li, attention_mask)
    out = mixture_of_sparse_attention(
        q, keys, values, sm_scale=head_dim ** -0.5, attention_dropout=0.0,
        sink_size=past_key_value.static_cache_size[li],
        local_size=past_key_value.circular_cache_size[li],
        head_start_index=past_key_value.cache_head_start_index[li],
        head_valid_length=past_key_value.cache_valid_length[li],
    )   # [batch, q_len, heads, head_dim]
    return attn.o_proj(out.reshape(bsz, q_len, num_heads * head_dim))


class LlamaMixtureAttention(nn.Module):
    """One attention layer.  ``forward`` follows the reference's (:232-326)."""

    def __init__(self, hidden_size: int, num_heads: int, num_key_value_heads: Optional[int] = None,
                 head_dim: Optional[int] = None, layer_idx: int = 0, bias: bool = False,
                 dtype: torch.dtype = torch.float16, device=None):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_key_value_heads = num_key_value_heads or num_heads
        assert num_heads % self.num_key_value_heads == 0
        self.num_key_value_groups = num_heads // self.num_key_value_heads
        self.head_dim = head_dim or hidden_size // num_heads
        self.layer_idx = layer_idx
        kw = dict(bias=bias, dtype=dtype, device=device)
        self.q_proj = nn.Linear(hidden_size, num_heads * self.head_dim, **kw)
        self.k_proj = nn.Linear(hidden_size, self.num_key_value_heads * self.head_dim, **kw)
        self.v_proj = nn.Linear(hidden_size, self.num_key_value_heads * self.head_dim, **kw)
        self.o_proj = nn.Linear(num_heads * self.head_dim, hidden_size, **kw)

    def forward(self, hidden_states: Tensor, position_embeddings: Tuple[Tensor, Tensor],
                past_key_value: StaticCircularCache, attention_mask: Optional[Tensor] = None) -> Tensor:
        """hidden_states ``[batch, q_len, hidden]``; position_embeddings ``(cos, sin)`` each
        ``[batch or 1, q_len, head_dim]``; attention_mask ``[batch, kv_len]`` of 0/1 marks left
        padding of a prompt.  Returns ``[batch, q_len, hidden]``."""
        return mixture_attention_forward(self, hidden_states, position_embeddings, past_key_value, attention_mask)


def install_plan(attention_layers: List[nn.Module], moa_config: Dict, permute_head: bool) -> Dict:
    """What ``set_mixture_of_attention`` does to the plan and the projections (reference :373-398):
    returns the plan as stored on the model (re-ordered like the heads when ``permute_head``)."""
    alphas = [list(a) for a in moa_config["alphas"]]
    betas = [list(b) for b in moa_config["betas"]]
    assert len(alphas) == len(attention_layers) and len(betas) == len(attention_layers)
    if permute_head:
        permutations, _ = moa_config_to_permutation({"alphas": alphas, "betas": betas})
        for layer, perm in zip(attention_layers, permutations):
            i = layer.layer_idx
            alphas[i] = [alphas[i][j] for j in perm.tolist()]
            betas[i] = [betas[i][j] for j in perm.tolist()]
            heads, hk, _ = attention_geometry(layer)
            g = heads // hk
            permute_attention_projection(layer.q_proj, perm, hk, g)
            permute_attention_projection(layer.k_proj, perm, hk)
            permute_attention_projection(layer.v_proj, perm, hk)
            permute_output_projection(layer.o_proj, perm, hk, g)
    return {"alphas": alphas, "betas": betas}


def new_cache_for_plan(moa_config: Dict, max_new_token: int, batch_size: int, seq_len: int, head_dim: int,
                       device, dtype, verbose: bool = False) -> StaticCircularCache:
    """The cache the reference's model forward builds at the start of a generation
    (modeling_llama.py:93-112): sizes from the plan at this prompt length.  ``verbose`` prints the
    cache-size summary, as the reference does when ``moa_verbose`` was set (:95-104)."""
    cfg = moa_config_to_cache_config(moa_config, seq_len, max_new_token=max_new_token, sink_size=64,
                                     minimum_cache_size=128, split_size=64, verbose=verbose)
    return StaticCircularCache(cache_size=cfg["cache_size"], static_size=cfg["static_size"], batch_size=batch_size,
                               head_dim=head_dim, device=device, dtype=dtype)


class LlamaMixtureAttentionStack(nn.Module):
    """The attention path of a decoder: ``num_layers`` attention layers with residual
    connections (norms and MLPs are not on the path and are left out).  Carries what
    ``set_mixture_of_attention`` sets up in the reference: the plan, the optional head
    permutation, and the cache built from the plan."""

    def __init__(self, num_layers: int, hidden_size: int, num_heads: int,
                 num_key_value_heads: Optional[int] = None, head_dim: Optional[int] = None,
                 rope_base: float = 10000.0, dtype: torch.dtype = torch.float16, device=None):
        super().__init__()
        self.layers = nn.ModuleList(
            LlamaMixtureAttention(hidden_size, num_heads, num_key_value_heads, head_dim, layer_idx=i, dtype=dtype,
                                  device=device) for i in range(num_layers))
        self.rope_base = rope_base
        self.dtype = dtype
        self.use_moa = False
        self.moa_config: Optional[Dict] = None
        self.moa_max_new_token = 1024
        self.eval()

    def set_mixture_of_attention(self, moa_config: Dict, permute_head: bool = False,
                                 moa_max_new_token: int = 1024) -> None:
        """Stores the plan (``alphas``/``betas`` per layer and kv head) and, with ``permute_head``,
        clusters heads with equal (alpha, beta): the plan and the q/k/v/o projections of every
        layer are re-ordered consistently (reference :373-398), which leaves the layer's function
        unchanged."""
        self.moa_config = install_plan(list(self.layers), moa_config, permute_head)
        self.moa_max_new_token = moa_max_new_token
        self.use_moa = True

    def new_cache(self, batch_size: int, seq_len: int, device) -> StaticCircularCache:
        """The cache the reference's model forward builds at the start of a generation
        (modeling_llama.py:93-112): sizes from the plan at this prompt length."""
        assert self.use_moa, "call set_mixture_of_attention first"
        return new_cache_for_plan(self.moa_config, self.moa_max_new_token, batch_size, seq_len,
                                  self.layers[0].head_dim, device, self.dtype)

    @torch.no_grad()
    def forward(self, hidden_states: Tensor, position_ids: Tensor, past_key_value: StaticCircularCache,
                attention_mask: Optional[Tensor] = None) -> Tensor:
        cos, sin = rotary_cos_sin(position_ids, self.layers[0].head_dim, self.dtype, self.rope_base)
        for layer in self.layers:
            hidden_states = hidden_states + layer(hidden_states, (cos, sin), past_key_value, attention_mask)
        return hidden_states


class LlamaRMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) * weight, the mean in fp32 (plain torch: not on the accelerated path)."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, dtype=torch.float16, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device))
        self.eps = eps

    def forward(self, x: Tensor) -> Tensor:
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).to(x.dtype) * self.weight


class LlamaMLP(nn.Module):
    """SwiGLU feed-forward (library GEMMs: not on the accelerated path).  Long prompts go through in
    slices of ``token_chunk`` tokens so that the intermediate stays small."""

    def __init__(self, hidden_size: int, intermediate_size: int, dtype=torch.float16, device=None,
                 token_chunk: int = 16384):
        super().__init__()
        kw = dict(bias=False, dtype=dtype, device=device)
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, **kw)
        self.token_chunk = token_chunk

    def forward(self, x: Tensor) -> Tensor:
        flat = x.reshape(-1, x.shape[-1])
        if flat.shape[0] <= self.token_chunk:
            return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))
        out = torch.empty_like(flat)
        for i in range(0, flat.shape[0], self.token_chunk):
            xs = flat[i:i + self.token_chunk]
            out[i:i + self.token_chunk] = self.down_proj(nn.functional.silu(self.gate_proj(xs)) * self.up_proj(xs))
        return out.view_as(x)


class LlamaMixtureDecoderLayer(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, num_key_value_heads: int, head_dim: int,
                 intermediate_size: int, layer_idx: int, rms_eps: float, dtype, device):
        super().__init__()
        self.input_layernorm = LlamaRMSNorm(hidden_size, rms_eps, dtype, device)
        self.self_attn = LlamaMixtureAttention(hidden_size, num_heads, num_key_value_heads, head_dim,
                                               layer_idx=layer_idx, dtype=dtype, device=device)
        self.post_attention_layernorm = LlamaRMSNorm(hidden_size, rms_eps, dtype, device)
        self.mlp = LlamaMLP(hidden_size, intermediate_size, dtype, device)

    def forward(self, hidden_states: Tensor, position_embeddings, past_key_value, attention_mask=None) -> Tensor:
        hidden_states = hidden_states + self.self_attn(self.input_layernorm(hidden_states), position_embeddings,
                                                       past_key_value, attention_mask)
        return hidden_states + self.mlp(self.post_attention_layernorm(hidden_states))


class LlamaMixtureForCausalLM(nn.Module):
    """A whole Llama-shaped decoder around the attention path, for end-to-end measurements with
    random weights: embedding, ``num_layers`` x (RMSNorm, attention, RMSNorm, SwiGLU), final norm,
    LM head.  Follows the reference's model forward (MoA/models/llama/modeling_llama.py:52-204): the
    cache is built from the plan at the first call of a generation, positions continue from the
    cache's length.  Only the attention goes through libmoa_hip.so; the rest is torch."""

    def __init__(self, num_layers: int, hidden_size: int, num_heads: int, num_key_value_heads: int,
                 intermediate_size: int, vocab_size: int, head_dim: Optional[int] = None,
                 rope_base: float = 10000.0, rms_eps: float = 1e-5, dtype: torch.dtype = torch.float16, device=None):
        super().__init__()
        head_dim = head_dim or hidden_size // num_heads
        self.embed_tokens = nn.Embedding(vocab_size, hidden_size, dtype=dtype, device=device)
        self.layers = nn.ModuleList(
            LlamaMixtureDecoderLayer(hidden_size, num_heads, num_key_value_heads, head_dim, intermediate_size, i,
                                     rms_eps, dtype, device) for i in range(num_layers))
        self.norm = LlamaRMSNorm(hidden_size, rms_eps, dtype, device)
        self.lm_head = nn.Linear(hidden_size, vocab_size, bias=False, dtype=dtype, device=device)
        self.head_dim = head_dim
        self.rope_base = rope_base
        self.dtype = dtype
        self.use_moa = False
        self.moa_config: Optional[Dict] = None
        self.moa_max_new_token = 1024
        self.eval()

    def set_mixture_of_attention(self, moa_config: Dict, permute_head: bool = False,
                                 moa_max_new_token: int = 1024) -> None:
        self.moa_config = install_plan([l.self_attn for l in self.layers], moa_config, permute_head)
        self.moa_max_new_token = moa_max_new_token
        self.use_moa = True

    @torch.no_grad()
    def forward(self, input_ids: Tensor, past_key_values: Optional[StaticCircularCache] = None,
                attention_mask: Optional[Tensor] = None, position_ids: Optional[Tensor] = None
                ) -> Tuple[Tensor, StaticCircularCache]:
        """input_ids ``[batch, q_len]``.  Returns the logits of the last position ``[batch, vocab]`` and
        the cache (created here when none is passed).  ``position_ids`` ``[1 or batch, q_len]`` default
        to the positions after the cache's length; a caller that replays a captured decode step passes
        a device tensor that it advances itself."""
        assert self.use_moa, "call set_mixture_of_attention first"
        bsz, q_len = input_ids.shape
        if past_key_values is None:
            past_key_values = new_cache_for_plan(self.moa_config, self.moa_max_new_token, bsz, q_len,
                                                 self.head_dim, input_ids.device, self.dtype)
        if position_ids is None:
            past = past_key_values.get_seq_length()
            position_ids = torch.arange(past, past + q_len, device=input_ids.device)[None, :]
        if attention_mask is not None and not (attention_mask == 0).any():
            attention_mask = None    # as the reference: a mask without padding is no mask (:119-121)
        cos_sin = rotary_cos_sin(position_ids, self.head_dim, self.dtype, self.rope_base)
        hidden_states = self.embed_tokens(input_ids)
        for layer in self.layers:
            hidden_states = layer(hidden_states, cos_sin, past_key_values, attention_mask)
        logits = self.lm_head(self.norm(hidden_states[:, -1, :]))
        return logits, past_key_values

    @torch.no_grad()
    def generate_greedy(self, input_ids: Tensor, max_new_tokens: int) -> Tensor:
        """Prompt, then ``max_new_tokens`` greedy steps.  Returns the new token ids ``[batch, max_new_tokens]``."""
        logits, cache = self.forward(input_ids)
        out = []
        for _ in range(max_new_tokens):
            nxt = logits.argmax(-1, keepdim=True)
            out.append(nxt)
            logits, cache = self.forward(nxt, cache)
        return torch.cat(out, dim=1)


# ---- binding the path into a transformers-style Llama model -------------------------------------------
# The reference patches a loaded transformers model in place: update_model_function (MoA/models/interface.py)
# binds set_mixture_of_attention to ``model.model``; calling it swaps in the model forward and the attention
# forwards below (MoA/models/llama/modeling_llama.py:334-406).  The same here, for any model whose
# ``model.model`` has ``embed_tokens``, ``layers[i].{input_layernorm, self_attn, post_attention_layernorm,
# mlp}``, ``norm`` and a ``config`` (a transformers LlamaModel of any recent release: only submodule names
# are relied on, not its internal mask and cache helpers, which changed between releases).


def _rope_base(config) -> float:
    params = getattr(config, "rope_parameters", None)
    if isinstance(params, dict) and "rope_theta" in params:
        kind = params.get("rope_type", "default")
        if kind != "default":
            raise NotImplementedError(f"rope_type {kind!r}: only the default rotary embedding is covered")
        return float(params["rope_theta"])
    if getattr(config, "rope_scaling", None):
        raise NotImplementedError("rope_scaling: only the default rotary embedding is covered")
    return float(getattr(config, "rope_theta", 10000.0))


def LlamaModel_MixtureAttention_forward(self, input_ids=None, attention_mask=None, position_ids=None,
                                        past_key_values=None, inputs_embeds=None, use_cache=None,
                                        output_attentions=None, output_hidden_states=None, return_dict=None,
                                        cache_position=None, **kwargs):
    """Model forward with the MoA attention path (reference modeling_llama.py:52-204): builds the
    StaticCircularCache from the plan at the first call of a generation (any other kind of cache passed
    in -- ``generate`` of transformers hands over its own empty one -- is replaced, as in the reference
    :93-112; the cache summary is printed when ``moa_verbose`` was set), continues the positions from the
    cache unless ``cache_position`` / ``position_ids`` say otherwise (:114-120), runs the decoder layers
    with the attention of ``mixture_attention_forward``.  Returns a ``BaseModelOutputWithPast`` with
    ``last_hidden_state`` (only the last position when ``last_hidden_only`` was set, :188-190),
    ``past_key_values`` (the StaticCircularCache) and, when asked for, ``hidden_states``; a tuple of the
    non-empty ones with ``return_dict=False`` (:183-184).  ``output_attentions`` raises, as in the
    reference (:126-129)."""
    assert self.use_moa, "call set_mixture_of_attention first"
    config = getattr(self, "config", None)
    if output_attentions is None:
        output_attentions = getattr(config, "output_attentions", False)
    if output_hidden_states is None:
        output_hidden_states = getattr(config, "output_hidden_states", False)
    if return_dict is None:
        return_dict = getattr(config, "use_return_dict", True)
    if output_attentions:
        raise NotImplementedError("output_attentions is not supported in mixture of attention")
    if (input_ids is None) == (inputs_embeds is None):
        raise ValueError("You must specify exactly one of input_ids or inputs_embeds")
    hidden_states = self.embed_tokens(input_ids) if inputs_embeds is None else inputs_embeds
    bsz, q_len = hidden_states.shape[:2]
    _, _, head_dim = attention_geometry(self.layers[0].self_attn)
    if not isinstance(past_key_values, StaticCircularCache):
        past_key_values = new_cache_for_plan(self.moa_config, self.moa_max_new_token, bsz, q_len, head_dim,
                                             hidden_states.device, hidden_states.dtype,
                                             verbose=getattr(self, "moa_verbose", False))
    if position_ids is None:
        if cache_position is None:
            past = past_key_values.get_seq_length()
            cache_position = torch.arange(past, past + q_len, device=hidden_states.device)
        position_ids = cache_position[None, :]
    # A mask without padding is no mask (:119-121).  A decode step needs none at all (the cache's decode
    # branch ignores it, cache_utils.py:1020-1058), so only a prompt pays for looking at it.
    if q_len == 1 or (attention_mask is not None and not (attention_mask == 0).any()):
        attention_mask = None
    cos_sin = rotary_cos_sin(position_ids, head_dim, hidden_states.dtype, _rope_base(self.config))
    all_hidden_states = () if output_hidden_states else None
    with torch.no_grad():
        for layer in self.layers:
            if output_hidden_states:
                all_hidden_states += (hidden_states,)
            residual = hidden_states
            hidden_states = residual + mixture_attention_forward(layer.self_attn, layer.input_layernorm(hidden_states),
                                                                 cos_sin, past_key_values, attention_mask)
            hidden_states = hidden_states + layer.mlp(layer.post_attention_layernorm(hidden_states))
        hidden_states = self.norm(hidden_states)
    if output_hidden_states:
        all_hidden_states += (hidden_states,)
    if not return_dict:
        return tuple(v for v in (hidden_states, past_key_values, all_hidden_states) if v is not None)
    if getattr(self, "last_hidden_only", False):
        hidden_states = hidden_states[:, -1:, :]
    try:
        from transformers.modeling_outputs import BaseModelOutputWithPast
        return BaseModelOutputWithPast(last_hidden_state=hidden_states, past_key_values=past_key_values,
                                       hidden_states=all_hidden_states)
    except ImportError:   # a duck-typed model without transformers installed
        from types import SimpleNamespace
        return SimpleNamespace(last_hidden_state=hidden_states, past_key_values=past_key_values,
                               hidden_states=all_hidden_states, attentions=None)


def LlamaModel_set_mixture_of_attention(self, moa_config: Dict, permute_head: bool = False, moa_verbose: bool = False,
                                        moa_max_new_token: int = 1024, last_hidden_only: bool = True,
                                        sparse_prefill: bool = True) -> None:
    """Same arguments as the reference's function of this name (modeling_llama.py:334-406): stores the
    plan, optionally clusters heads with equal (alpha, beta) by permuting the plan and the q/k/v/o
    projections of every layer, and swaps in the MoA model forward."""
    from types import MethodType

    assert sparse_prefill, "only support sparse prefill now"
    for i, layer in enumerate(self.layers):
        if getattr(layer.self_attn, "layer_idx", None) is None:
            layer.self_attn.layer_idx = i
    plan = {"alphas": [list(a) for a in moa_config["alphas"]], "betas": [list(b) for b in moa_config["betas"]]}
    self.moa_config = install_plan([layer.self_attn for layer in self.layers], plan, permute_head)
    self.moa_verbose = moa_verbose
    self.last_hidden_only = last_hidden_only
    self.moa_max_new_token = moa_max_new_token
    self.use_moa = True
    self.forward = MethodType(LlamaModel_MixtureAttention_forward, self)
    self.eval()


def LlamaModel_use_block_sparse_attention_lut(self, *args, **kwargs):
    """The reference's older lookup-table sparse attention (deprecated there); not part of this path."""
    raise NotImplementedError("the lookup-table sparse attention is not part of this build; use set_mixture_of_attention")
