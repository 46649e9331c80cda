"""Gated DeltaNet layer: projections, causal short convolutions, the gated delta rule, gated RMS
norm, output projection - the immediate caller of this package's kernels, with the constructor arguments,
parameter names (so upstream checkpoints load with ``load_state_dict``) and call signature of the reference's
``GatedDeltaNet`` (fla/layers/gated_deltanet.py:28-364), and its cache contract: ``past_key_values[layer_idx]``
is a dict with ``recurrent_state`` ``[N, HV, V, K]`` fp32 and ``conv_state`` (three ``[N, D, W]`` tensors);
``past_key_values.update(layer_idx=..., recurrent_state=..., conv_state=..., offset=...)`` stores them
(fla/layers/utils.py:271-293, fla/models/utils.py:42-118).  ``LayerCache`` is a minimal cache with that contract;
upstream's ``fla.models.utils.Cache`` objects are used the same way.

Prompts longer than 64 tokens run the chunk kernels, shorter calls (decode) the token recurrence; both read and
write the same state layout, so a prefill hands over to decode through the cache without any conversion.
The linear projections are torch matmuls; everything between them runs in this package's HIP kernels.
In training mode (``.train()``) the call is differentiable: the convolutions, the chunked operator and the gated norm
each have backward kernels, and every call runs the chunk kernels as in the reference (fla/layers/gated_deltanet.py:237-239).
In eval mode no autograd graph is built (the token recurrence of decode has no backward)."""
from __future__ import annotations

import math
import warnings

import torch
import torch.nn as nn
import torch.nn.functional as F

from fla_hip.modules import FusedRMSNormGated, ShortConvolution
from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule


class LayerCache:
    """Per-layer states of a stack of layers: ``cache[i]`` is layer i's dict, ``update`` replaces entries in it."""

    def __init__(self):
        self.states: list[dict] = []
        self._seen_tokens = 0

    def __len__(self) -> int:
        return len(self.states)

    def __getitem__(self, layer_idx: int) -> dict:
        return self.states[layer_idx]

    def update(self, *, layer_idx: int, recurrent_state=None, conv_state=None, offset: int = 1, **_) -> dict:
        while len(self.states) <= layer_idx:
            self.states.append(dict(recurrent_state=None, attn_state=None, conv_state=None, ffn_state=None))
        entry = self.states[layer_idx]
        if recurrent_state is not None:
            entry['recurrent_state'] = recurrent_state
        if conv_state is not None:
            entry['conv_state'] = conv_state
        if layer_idx == 0:
            self._seen_tokens += offset
        return entry

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self._seen_tokens if len(self.states) > layer_idx else 0


def _unpad(hidden_states, attention_mask, q_len):
    """[B, T, ...] with a 0/1 mask -> ([1, total, ...], flat indices of the kept tokens, cu_seqlens)."""
    mask = attention_mask[:, -q_len:].to(torch.bool)
    lens = mask.sum(-1, dtype=torch.int32)
    cu_seqlens = F.pad(lens.cumsum(0, dtype=torch.int32), (1, 0))
    indices = mask.flatten().nonzero(as_tuple=False).flatten()
    flat = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return flat.index_select(0, indices).unsqueeze(0), indices, cu_seqlens


class GatedDeltaNet(nn.Module):

    def __init__(
        self,
        hidden_size: int = 2048,
        expand_v: float = 2,
        head_dim: int = 256,
        num_heads: int = 6,
        num_v_heads: int | None = None,
        mode: str = 'chunk',
        use_gate: bool = True,
        use_short_conv: bool = True,
        allow_neg_eigval: bool = False,
        conv_size: int = 4,
        conv_bias: bool = False,
        layer_idx: int | None = None,
        norm_eps: float = 1e-5,
        **kwargs,
    ):
        super().__init__()
        assert mode in ['chunk', 'fused_recurrent'], f'Not supported mode `{mode}`.'
        self.mode, self.allow_neg_eigval, self.hidden_size, self.expand_v = mode, allow_neg_eigval, hidden_size, expand_v
        self.use_gate, self.use_short_conv, self.conv_size, self.conv_bias = use_gate, use_short_conv, conv_size, conv_bias
        self.head_dim = self.head_k_dim = head_dim
        self.num_heads = num_heads
        self.num_v_heads = num_heads if num_v_heads is None else num_v_heads
        self.head_v_dim = int(head_dim * expand_v)
        self.key_dim = num_heads * head_dim
        self.value_dim = self.num_v_heads * self.head_v_dim
        self.layer_idx = layer_idx
        if not math.isclose(head_dim * expand_v, self.head_v_dim, rel_tol=1e-5):
            raise ValueError(f'expand_v={expand_v} times head_dim={head_dim} is not an integer head size')
        if self.num_v_heads > num_heads and self.num_v_heads % num_heads != 0:
            raise ValueError(f'num_v_heads={self.num_v_heads} must be divisible by num_heads={num_heads}.')

        self.q_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.k_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.v_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
        self.a_proj = nn.Linear(hidden_size, self.num_v_heads, bias=False)
        self.b_proj = nn.Linear(hidden_size, self.num_v_heads, bias=False)
        # decay rate and step-size bias per value head, initialised as the reference does (:153-170)
        self.A_log = nn.Parameter(torch.log(torch.empty(self.num_v_heads, dtype=torch.float32).uniform_(0, 16)))
        dt = torch.exp(torch.rand(self.num_v_heads) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
        self.dt_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))           # inverse of softplus
        self.A_log._no_weight_decay = self.dt_bias._no_weight_decay = True
        if use_short_conv:
            self.q_conv1d = ShortConvolution(self.key_dim, conv_size, bias=conv_bias, activation='silu')
            self.k_conv1d = ShortConvolution(self.key_dim, conv_size, bias=conv_bias, activation='silu')
            self.v_conv1d = ShortConvolution(self.value_dim, conv_size, bias=conv_bias, activation='silu')
        else:
            warnings.warn('ShortConvolution is crucial to the performance. Do not turn it off, i.e., setting '
                          '`use_short_conv=False` unless you know what you are doing.')
        if use_gate:
            self.g_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
            self.o_norm = FusedRMSNormGated(self.head_v_dim, eps=norm_eps)
        else:
            self.o_norm = nn.RMSNorm(self.head_v_dim, eps=norm_eps, dtype=torch.float32)
        self.o_proj = nn.Linear(self.value_dim, hidden_size, bias=False)

    def forward(
        self,
        hidden_states: torch.Tensor,
        attention_mask: torch.Tensor | None = None,
        past_key_values=None,
        use_cache: bool | None = False,
        output_attentions: bool | None = False,
        **kwargs,
    ):
        if self.training:
            return self._forward(hidden_states, attention_mask, past_key_values, use_cache, **kwargs)
        with torch.no_grad():
            return self._forward(hidden_states, attention_mask, past_key_values, use_cache, **kwargs)

    def _forward(self, hidden_states, attention_mask, past_key_values, use_cache, **kwargs):
        if attention_mask is not None:
            assert attention_mask.dim() == 2, 'attention_mask must be a 0-1 matrix [batch_size, seq_len] (0 = padding)'
        if past_key_values is not None and self.layer_idx is None:
            raise ValueError(f'{self.__class__.__name__} requires `layer_idx` when `past_key_values` is provided.')
        batch_size, q_len, _ = hidden_states.shape
        mode = 'fused_recurrent' if (q_len <= 64 and not self.training) else self.mode
        if self.training and mode != 'chunk':
            raise AssertionError('Only chunk mode is supported in training.')

        last_state = None
        if past_key_values is not None and len(past_key_values) > self.layer_idx:
            last_state = past_key_values[self.layer_idx]
        cu_seqlens, indices = kwargs.get('cu_seqlens'), None
        if cu_seqlens is None and attention_mask is not None:
            hidden_states, indices, cu_seqlens = _unpad(hidden_states, attention_mask, q_len)

        q, k, v = self.q_proj(hidden_states), self.k_proj(hidden_states), self.v_proj(hidden_states)
        conv_state = None
        if self.use_short_conv:
            cq, ck, cv = last_state['conv_state'] if last_state is not None and last_state.get('conv_state') is not None else (None,) * 3
            q, cq = self.q_conv1d(x=q, cache=cq, output_final_state=use_cache, cu_seqlens=cu_seqlens)
            k, ck = self.k_conv1d(x=k, cache=ck, output_final_state=use_cache, cu_seqlens=cu_seqlens)
            v, cv = self.v_conv1d(x=v, cache=cv, output_final_state=use_cache, cu_seqlens=cu_seqlens)
            conv_state = (cq, ck, cv)
        else:
            q, k, v = F.silu(q), F.silu(k), F.silu(v)
        q = q.unflatten(-1, (self.num_heads, self.head_k_dim))
        k = k.unflatten(-1, (self.num_heads, self.head_k_dim))
        v = v.unflatten(-1, (self.num_v_heads, self.head_v_dim))

        recurrent_state = last_state['recurrent_state'] if last_state is not None else None
        op = chunk_gated_delta_rule if mode == 'chunk' else fused_recurrent_gated_delta_rule
        extra = {}
        if (mode == 'fused_recurrent' and use_cache and recurrent_state is not None and recurrent_state.dtype == torch.float32
                and recurrent_state.is_contiguous()):
            # decode: the cached state is updated where it is - no allocation per step, and a step captured in a
            # HIP graph keeps reading and writing the same buffers on every replay
            extra['inplace_final_state'] = True
        o, recurrent_state = op(
            q=q, k=k, v=v, g=self.a_proj(hidden_states), beta=self.b_proj(hidden_states),
            A_log=self.A_log, dt_bias=self.dt_bias, initial_state=recurrent_state, output_final_state=use_cache,
            use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True,
            allow_neg_eigval=self.allow_neg_eigval, state_v_first=True, cu_seqlens=cu_seqlens, **extra)

        if past_key_values is not None:
            past_key_values.update(layer_idx=self.layer_idx, recurrent_state=recurrent_state,
                                   conv_state=conv_state if self.use_short_conv else None, offset=q_len)
        if self.use_gate:
            o = self.o_norm(o, self.g_proj(hidden_states).unflatten(-1, (self.num_v_heads, self.head_v_dim)))
        else:
            o = self.o_norm(o.float()).to(o.dtype)
        o = self.o_proj(o.flatten(-2))
        if indices is not None:                               # back to the padded [B, T, hidden] layout
            padded = o.new_zeros(batch_size * q_len, o.shape[-1])
            padded[indices] = o.squeeze(0)
            o = padded.view(batch_size, q_len, -1)
        return o, None, past_key_values
