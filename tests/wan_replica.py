"""A small stand-in for the diffusers Wan2.1 transformer, for tests (diffusers is not installed here).

Same module names, parameter layout and forward arithmetic as the model the reference's adapters wrap:
blocks with ``norm1 / attn1 / norm2 / attn2 / norm3 / ffn / scale_shift_table``, attention modules with
``to_q / to_k / to_v / to_out / norm_q / norm_k`` called by a processor in the order of
dax/adapters/wan/attn_adapter.py:76-100, a feed-forward ``net = [GELU(proj, approximate="tanh"), Dropout,
Linear]``, and the ``condition_embedder`` / ``proj_out`` subtrees that stay unquantised.
"""
import torch
import torch.nn.functional as F
from torch import nn


class FP32LayerNorm(nn.LayerNorm):
    def forward(self, x):
        return F.layer_norm(x.float(), self.normalized_shape, self.weight.float() if self.weight is not None else None,
                            self.bias.float() if self.bias is not None else None, self.eps).to(x.dtype)


class RMSNorm(nn.Module):
    def __init__(self, dim, eps=1e-6):
        super().__init__()
        self.weight, self.eps = nn.Parameter(torch.ones(dim)), eps

    def forward(self, x):
        v = x.float().pow(2).mean(-1, keepdim=True)
        return (x.float() * torch.rsqrt(v + self.eps)).to(x.dtype) * self.weight


def processor(attn, hidden_states, encoder_hidden_states=None, rotary_emb=None):
    if encoder_hidden_states is None:
        encoder_hidden_states = hidden_states
    query = attn.norm_q(attn.to_q(hidden_states))
    key = attn.norm_k(attn.to_k(encoder_hidden_states))
    value = attn.to_v(encoder_hidden_states)
    query = query.unflatten(2, (attn.heads, -1)).transpose(1, 2)
    key = key.unflatten(2, (attn.heads, -1)).transpose(1, 2)
    value = value.unflatten(2, (attn.heads, -1)).transpose(1, 2)
    out = F.scaled_dot_product_attention(query, key, value)
    out = out.transpose(1, 2).flatten(2, 3).type_as(query)
    out = attn.to_out[0](out)
    return attn.to_out[1](out)


class Attention(nn.Module):
    def __init__(self, dim, heads):
        super().__init__()
        self.heads = heads
        self.to_q, self.to_k, self.to_v = nn.Linear(dim, dim), nn.Linear(dim, dim), nn.Linear(dim, dim)
        self.to_out = nn.ModuleList([nn.Linear(dim, dim), nn.Dropout(0.0)])
        self.norm_q, self.norm_k = RMSNorm(dim), RMSNorm(dim)
        self.add_k_proj = None

    def forward(self, hidden_states, encoder_hidden_states=None, rotary_emb=None):
        return processor(self, hidden_states, encoder_hidden_states, rotary_emb)


class GELU(nn.Module):
    def __init__(self, dim, inner, approximate="tanh"):
        super().__init__()
        self.proj, self.approximate = nn.Linear(dim, inner), approximate

    def forward(self, x):
        return F.gelu(self.proj(x), approximate=self.approximate)


class FeedForward(nn.Module):
    def __init__(self, dim, inner):
        super().__init__()
        self.net = nn.ModuleList([GELU(dim, inner), nn.Dropout(0.0), nn.Linear(inner, dim)])

    def forward(self, x):
        for m in self.net:
            x = m(x)
        return x


class Block(nn.Module):
    def __init__(self, dim, ffn_dim, heads, eps=1e-6, cross_attn_norm=True):
        super().__init__()
        self.norm1 = FP32LayerNorm(dim, eps, elementwise_affine=False)
        self.attn1 = Attention(dim, heads)
        self.attn2 = Attention(dim, heads)
        self.norm2 = FP32LayerNorm(dim, eps, elementwise_affine=True) if cross_attn_norm else nn.Identity()
        self.ffn = FeedForward(dim, ffn_dim)
        self.norm3 = FP32LayerNorm(dim, eps, elementwise_affine=False)
        self.scale_shift_table = nn.Parameter(torch.randn(1, 6, dim) / dim ** 0.5)

    def forward(self, hidden_states, encoder_hidden_states, temb, rotary_emb=None):
        shift_msa, scale_msa, gate_msa, c_shift_msa, c_scale_msa, c_gate_msa = (
            self.scale_shift_table + temb.float()).chunk(6, dim=1)
        norm_hidden_states = (self.norm1(hidden_states.float()) * (1 + scale_msa) + shift_msa).type_as(hidden_states)
        attn_output = self.attn1(hidden_states=norm_hidden_states, rotary_emb=rotary_emb)
        hidden_states = (hidden_states.float() + attn_output * gate_msa).type_as(hidden_states)
        norm_hidden_states = self.norm2(hidden_states.float()).type_as(hidden_states)
        attn_output = self.attn2(hidden_states=norm_hidden_states, encoder_hidden_states=encoder_hidden_states)
        hidden_states = hidden_states + attn_output
        norm_hidden_states = (self.norm3(hidden_states.float()) * (1 + c_scale_msa) + c_shift_msa).type_as(hidden_states)
        ff_output = self.ffn(norm_hidden_states)
        hidden_states = (hidden_states.float() + ff_output.float() * c_gate_msa).type_as(hidden_states)
        return hidden_states


class Transformer(nn.Module):
    def __init__(self, dim=256, ffn_dim=512, heads=4, layers=2, cross_attn_norm=True):
        super().__init__()
        self.condition_embedder = nn.Sequential(nn.Linear(dim, dim), nn.SiLU(), nn.Linear(dim, 6 * dim))
        self.blocks = nn.ModuleList([Block(dim, ffn_dim, heads, cross_attn_norm=cross_attn_norm) for _ in range(layers)])
        self.proj_out = nn.Linear(dim, 64)
        self.dim = dim

    def forward(self, hidden_states, encoder_hidden_states, t):
        temb = self.condition_embedder(t).unflatten(1, (6, -1))
        for block in self.blocks:
            hidden_states = block(hidden_states, encoder_hidden_states, temb)
        return self.proj_out(hidden_states)
