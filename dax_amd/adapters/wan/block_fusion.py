"""Quantise once, where the activation is produced: block-level fusion for a quantised Wan2.1 DiT.

After ``quantize_transformer`` every projection of a DiT block quantises its own input.  Run eagerly
that costs, per block, three quantisations of the same self-attention input (to_q / to_k / to_v, the
reference calls them one after the other, dax/adapters/wan/attn_adapter.py:78-80), and a bf16 round
trip between each producer (adaLN-modulated LayerNorm, cross-attention LayerNorm, GELU) and the
quantiser behind it.  The reference leaves those fusions to ``torch.compile``
(dax/adapters/wan/functional.py:33-36); here they are explicit:

* ``fuse_transformer_blocks(transformer)`` rebinds the forward of every block whose linears are
  quantised so that
    - norm1 + modulation + quantisation is one kernel whose result feeds to_q, to_k and to_v,
    - norm2 (affine LayerNorm) + quantisation is one kernel in front of the cross-attention to_q,
    - the text-encoder states are quantised once for the cross-attention to_k and to_v,
    - norm3 + modulation + quantisation is one kernel in front of the FFN,
    - GELU-tanh + quantisation is one kernel between the two FFN linears.
  The block arithmetic is that of the diffusers ``WanTransformerBlock`` the reference runs
  (fp32 LayerNorm, ``norm(x) * (1 + scale) + shift`` cast back to bf16 -- the same operation order as
  dax/adapters/wan/transformer_adapter.py:151-153 -- gated residuals in fp32); attention itself is
  untouched: the processor receives a ``QuantizedActivation`` in place of the bf16 tensor and only
  hands it to the three projections.
* ``share_input_quant(linears)`` and ``fuse_linears(linears)`` are the two building blocks for other
  callers: one quantisation shared by linears that read the same tensor, and the N-concatenated
  single linear (bit-identical outputs, one GEMM launch).
"""
from __future__ import annotations

import types
import weakref
from typing import Optional, Sequence

import torch
from torch import Tensor, nn

from ... import ops
from ...quant.nn.dynamic.linear import Linear, QuantizedActivation

_FMT = {torch.int8: "i8", torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}


# ----------------------------------------------------------------------------- building blocks
def layernorm_quant(x: Tensor, mul: Optional[Tensor], add: Optional[Tensor], eps: float,
                    like: Linear) -> QuantizedActivation:
    """``bf16(layer_norm_f32(x) * mul + add)`` quantised for ``like``.  x [B, S, K] (or [M, K]);
    mul / add broadcastable to [B, 1, K] (one vector pair per batch element) or None."""
    k = x.shape[-1]
    flat = x.reshape(-1, k)
    batch = x.shape[0] if x.dim() == 3 else 1
    rows_per_group = flat.shape[0] // batch if batch else 1

    def vec(v):
        if v is None:
            return None
        return v.to(torch.float32).expand(batch, 1, k).reshape(batch, k).contiguous() if x.dim() == 3 \
            else v.to(torch.float32).reshape(1, k).contiguous()

    fn = getattr(ops, "layernorm_act_quant_" + _FMT[like.input_dtype])
    xq, sx, _ = fn(flat, vec(mul), vec(add), max(1, rows_per_group), eps)
    return QuantizedActivation(xq, sx, x.shape[:-1], k, like.input_dtype)


def gelu_tanh_quant(x: Tensor, like: Linear) -> QuantizedActivation:
    """``bf16(gelu(x, approximate="tanh"))`` quantised for ``like``."""
    k = x.shape[-1]
    xq, sx, _ = getattr(ops, "gelu_tanh_act_quant_" + _FMT[like.input_dtype])(x.reshape(-1, k))
    return QuantizedActivation(xq, sx, x.shape[:-1], k, like.input_dtype)


class _SharedQuant:
    """Remembers the quantised form of the last tensor seen.  A hit needs the same tensor object (held
    through a weak reference, so a new tensor that reuses a freed address cannot match) at the same
    version counter (any in-place write since then misses)."""

    def __init__(self):
        self.ref, self.version, self.dtype, self.qa = None, None, None, None

    def get(self, lin: Linear, x: Tensor) -> QuantizedActivation:
        hit = self.ref is not None and self.ref() is x and self.version == x._version and self.dtype == lin.input_dtype
        if not hit:
            self.qa = lin.quantize_activation(x)
            self.ref, self.version, self.dtype = weakref.ref(x), x._version, lin.input_dtype
        return self.qa

    def clear(self):
        self.ref, self.version, self.dtype, self.qa = None, None, None, None


def share_input_quant(linears: Sequence[Linear]) -> _SharedQuant:
    """Makes ``linears`` (same in_features and activation dtype) quantise a tensor once when they are
    called with the same tensor one after the other, as the attention processor does with q / k / v.
    Outputs are bit-identical to the separate calls.  Returns the cache (``clear()`` drops its tensor)."""
    first = linears[0]
    for lin in linears:
        if not isinstance(lin, Linear) or lin.in_features != first.in_features or lin.input_dtype != first.input_dtype:
            raise ValueError("share_input_quant needs quantised linears with the same in_features and activation dtype")
    cache = _SharedQuant()
    for lin in linears:
        plain = lin.forward

        def forward(self, input, _plain=plain):
            if isinstance(input, Tensor):
                input = cache.get(self, input)
            return _plain(input)

        lin.forward = types.MethodType(forward, lin)
    return cache


@torch.no_grad()
def fuse_linears(linears: Sequence[Linear]) -> Linear:
    """One quantised linear whose output is the concatenation of the outputs of ``linears`` along the
    last dimension (e.g. q | k | v: 5120 -> 15360).  Per-channel weight scales make this exact."""
    first = linears[0]
    for lin in linears:
        if (not isinstance(lin, Linear) or lin.in_features != first.in_features or lin.input_dtype != first.input_dtype
                or lin.weight_dtype != first.weight_dtype or (lin.bias is None) != (first.bias is None)
                or lin.act_scale_fp32 != first.act_scale_fp32):
            raise ValueError("fuse_linears needs quantised linears of one kind reading the same input")
    n = sum(lin.out_features for lin in linears)
    fused = Linear(first.in_features, n, first.bias is not None, first.qweight.device, first.weight_dtype,
                   first.input_dtype, first.out_dtype, first.weight_qscheme, first.input_qscheme)
    fused.qweight = torch.cat([lin.qweight.view(torch.uint8) for lin in linears], 0).view(first.qweight.dtype)
    fused.weight_scale = torch.cat([lin.weight_scale for lin in linears], 1)
    if first.bias is not None:
        fused.bias = nn.Parameter(torch.cat([lin.bias.detach() for lin in linears], 0), requires_grad=False)
    if first.act_scale_fp32:
        fused.act_scale_fp32 = True
    fused.refresh_derived()
    return fused


# ----------------------------------------------------------------------------- FFN
class GeluTanhQuant(nn.Module):
    """Stands in for the FFN's ``GELU(approximate="tanh")`` projection module: proj, then GELU and the
    quantisation for the next linear in one kernel."""

    def __init__(self, proj: nn.Module, consumer: Linear):
        super().__init__()
        self.proj = proj
        self._consumer = [consumer]      # not a sub-module: it stays where it is in the FFN

    def forward(self, hidden_states):
        return gelu_tanh_quant(self.proj(hidden_states), self._consumer[0])


def _fuse_ffn(ffn) -> bool:
    net = getattr(ffn, "net", None)
    if net is None or len(net) != 3:
        return False
    act, drop, out = net[0], net[1], net[2]
    if not (isinstance(out, Linear) and hasattr(act, "proj") and getattr(act, "approximate", None) == "tanh"):
        return False
    if isinstance(drop, nn.Dropout) and drop.p != 0.0:
        return False
    net[0] = GeluTanhQuant(act.proj, out)
    net[1] = nn.Identity()
    return True


# ----------------------------------------------------------------------------- block
def _ln_eps(norm) -> float:
    return float(getattr(norm, "eps", 1e-6))


def _fused_block_forward(self, hidden_states: Tensor, encoder_hidden_states: Tensor, temb: Tensor, rotary_emb=None):
    shift_msa, scale_msa, gate_msa, c_shift_msa, c_scale_msa, c_gate_msa = (
        self.scale_shift_table + temb.float()).chunk(6, dim=1)

    # 1. self-attention: norm1 + modulation + quantisation, shared by to_q / to_k / to_v
    qa = layernorm_quant(hidden_states, 1 + scale_msa, shift_msa, _ln_eps(self.norm1), self.attn1.to_q)
    attn_output = self.attn1(hidden_states=qa, rotary_emb=rotary_emb)
    hidden_states = (hidden_states.float() + attn_output * gate_msa).type_as(hidden_states)

    # 2. cross-attention: affine LayerNorm + quantisation in front of to_q (identity norm: plain quantiser)
    if isinstance(self.norm2, nn.LayerNorm):
        w = self.norm2.weight.float().reshape(1, 1, -1) if self.norm2.weight is not None else None
        b = self.norm2.bias.float().reshape(1, 1, -1) if self.norm2.bias is not None else None
        qa = layernorm_quant(hidden_states, w, b, _ln_eps(self.norm2), self.attn2.to_q)
    else:
        qa = self.attn2.to_q.quantize_activation(self.norm2(hidden_states))
    attn_output = self.attn2(hidden_states=qa, encoder_hidden_states=encoder_hidden_states)
    hidden_states = hidden_states + attn_output

    # 3. feed-forward: norm3 + modulation + quantisation; GELU + quantisation sits inside the FFN
    qa = layernorm_quant(hidden_states, 1 + c_scale_msa, c_shift_msa, _ln_eps(self.norm3), self._daxq_ffn_in)
    ff_output = self.ffn(qa)
    hidden_states = (hidden_states.float() + ff_output.float() * c_gate_msa).type_as(hidden_states)
    return hidden_states


def _block_is_fusable(block) -> bool:
    a1, a2, ffn = getattr(block, "attn1", None), getattr(block, "attn2", None), getattr(block, "ffn", None)
    if a1 is None or a2 is None or ffn is None or not hasattr(block, "scale_shift_table"):
        return False
    lins = [getattr(a1, n, None) for n in ("to_q", "to_k", "to_v")] + [getattr(a2, n, None) for n in ("to_q", "to_k", "to_v")]
    if not all(isinstance(l, Linear) for l in lins):
        return False
    if any(l.act_scale_fp32 for l in lins):  # the fused producer kernels round the scale as the eager chain does
        return False
    net = getattr(ffn, "net", None)
    first = getattr(net[0], "proj", None) if net is not None and len(net) else None
    return isinstance(first, Linear) and not any(getattr(n, "elementwise_affine", False) for n in (block.norm1, block.norm3))


def fuse_transformer_blocks(transformer) -> int:
    """Applies the block-level fusion to every block of ``transformer.blocks`` whose projections are
    quantised ``Linear`` modules.  Returns the number of blocks changed; blocks of another shape are left
    as they are."""
    done = 0
    for block in getattr(transformer, "blocks", []):
        if getattr(block, "_daxq_fused", False) or not _block_is_fusable(block):
            continue
        object.__setattr__(block, "_daxq_ffn_in", block.ffn.net[0].proj)  # plain attribute, not a second registration
        _fuse_ffn(block.ffn)
        share_input_quant([block.attn2.to_k, block.attn2.to_v])
        block.forward = types.MethodType(_fused_block_forward, block)
        object.__setattr__(block, "_daxq_fused", True)
        done += 1
    return done
