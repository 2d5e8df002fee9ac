"""Attention whose keys and values are read out of one small latent per token.

For a token at position ``p`` with input ``h`` (``H`` heads; per head ``D`` unrotated and ``R`` rotated query/key
elements and ``Dv`` value elements; latent widths ``rq`` and ``r``):

    c_q = rms(W_dq h) * g_q                         [rq]
    q_h = (W_uq c_q)_h = [q_h^plain (D) | q_h^rot (R)]
    [a (r) | b (R)] = W_dkv h
    c = rms(a) * g_kv                               the latent: all that is kept of the token, with
    k^rot = rotate(b, p)                            one rotated key part that every head shares
    k_h^plain = W_uk,h c        v_h = W_uv,h c
    score_h(p, j) = (q_h^plain . k_h^plain(j) + rotate(q_h^rot, p) . k^rot(j)) * scale        j <= p
    weights: softmax over j with one more term exp(sink_h) in the denominator
    y = W_o concat_h(sum_j weight_h(p, j) v_h(j))

Only ``c`` and ``k^rot`` are cached: a page row holds ``[c | k^rot]`` as the one key of the position and ``c`` as its
one value.  The readout matrices are moved to the query's side of the products, which changes nothing but the
order of the sums: ``q_h^plain . (W_uk,h c) = (W_uk,h^T q_h^plain) . c`` and ``sum_j w_j W_uv,h c_j = W_uv,h sum_j
w_j c_j``.  So every head asks the page attention with a query ``[W_uk,h^T q_h^plain | rotate(q_h^rot)]`` of width
``r + R`` over one shared key/value head, and its result (width ``r``) goes through ``W_uv,h``.

The rotation turns neighbouring pairs ``(2i, 2i + 1)`` of the first ``rotary_dim`` of the ``R`` elements.  A mixer
with ``kv_from_layer`` has no ``W_dkv`` and reads the pages that the named layer's latest run wrote.
"""

from __future__ import annotations

import torch

from .attention import _shared_position_encoding
from .plan import PagedKVNeed, TensorSpec
from .registry import register_mixer


@register_mixer("latent_attention")
class LatentAttention:
    """params: hidden_size, num_heads, head_dim (unrotated), rot_dim, value_head_dim, q_rank, kv_rank, scale,
    norm_eps, position (``{"kind", "params"}``, a rotary kind with ``pairing: "interleaved"``), and optionally sink
    (default False) and kv_from_layer."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.head_dim = int(params["head_dim"])
        self.rot_dim = int(params["rot_dim"])
        self.value_dim = int(params["value_head_dim"])
        self.q_rank = int(params["q_rank"])
        self.kv_rank = int(params["kv_rank"])
        self.scale = float(params["scale"])
        self.eps = float(params["norm_eps"])
        self.sink = bool(params.get("sink", False))
        self.kv_from_layer = params.get("kv_from_layer")
        self.position = _shared_position_encoding(params["position"], env)
        if self.position.rotary_dim > self.rot_dim or getattr(self.position, "pairing", "half") != "interleaved":
            raise ValueError("latent attention rotates neighbouring pairs of at most rot_dim elements")
        self.key_dim = self.kv_rank + self.rot_dim     # a cached key row: the latent and the shared rotated part
        check = getattr(env.kernels, "check_attention_geometry", None)
        if check is not None:
            check(self.num_heads, 1, self.key_dim, own_writer=True)
        page_dim = getattr(env.kernels, "attention_page_dim", None)
        self.page_dim = page_dim(self.key_dim, self.kv_rank, env.dtype) if page_dim is not None else None
        self.env = env
        self.w_down = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = None
        self.q_gain = self.kv_gain = self.sinks = None

    takes_scaled_rows = False

    @property
    def writes_kv(self) -> bool:
        return self.kv_from_layer is None

    def weight_specs(self):
        H = self.num_heads
        specs = {"dq": TensorSpec((self.q_rank, self.hidden)), "dq_norm": TensorSpec((self.q_rank,), "vector"),
                 "uq": TensorSpec((H * (self.head_dim + self.rot_dim), self.q_rank)),
                 "uk": TensorSpec((H * self.head_dim, self.kv_rank)), "uv": TensorSpec((H * self.value_dim, self.kv_rank)),
                 "o": TensorSpec((self.hidden, H * self.value_dim))}
        if self.writes_kv:
            specs["dkv"] = TensorSpec((self.key_dim, self.hidden))
            specs["dkv_norm"] = TensorSpec((self.kv_rank,), "vector")
        if self.sink:
            specs["sink"] = TensorSpec((H,), "vector")
        return specs

    def bind(self, tensors):
        H = self.num_heads
        down = [tensors["dq"], tensors["dkv"]] if self.writes_kv else [tensors["dq"]]
        self.w_down = torch.cat(down, dim=0).contiguous()
        self.w_uq = tensors["uq"].contiguous()
        # per head, as the matrix of a product x W^T: [kv_rank, head_dim] takes a head's plain query to the latent's side
        self.w_uk_t = tensors["uk"].view(H, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors["uv"].view(H, self.value_dim, self.kv_rank).contiguous()
        self.w_o = tensors["o"].contiguous()
        self.q_gain = tensors["dq_norm"].contiguous()
        self.kv_gain = tensors["dkv_norm"].contiguous() if self.writes_kv else None
        self.sinks = tensors["sink"].contiguous() if self.sink else None
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:
            prepare(self.w_o)

    def cache_need(self):
        if self.page_dim is not None:
            return PagedKVNeed(1, self.page_dim)
        return PagedKVNeed(1, self.key_dim, None, self.kv_rank)

    def state_need(self):
        return None

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        cos, sin = self.position.tables()
        rotary = self.position.rotary_dim
        width = self.page_dim or self.key_dim      # of a query as the page attention takes it
        proj = k.linear(h, self.w_down)
        cq = k.latent_prepare(proj, self.q_rank, self.q_gain, self.kv_rank if self.writes_kv else 0, self.kv_gain,
                              self.rot_dim, rotary, cos, sin, self.eps, ctx, cache, self.page_dim)
        q = k.linear(cq, self.w_uq)
        qa = k.headwise_linear(q, self.w_uk_t, self.head_dim + self.rot_dim, width, tail=self.rot_dim,
                               rotation=(rotary, cos, sin, ctx.positions))
        if self.page_dim is None:
            out = k.paged_attention(qa, self.num_heads, 1, self.key_dim, self.scale, None, ctx, cache,
                                    value_dim=self.kv_rank, sinks=self.sinks)
            out_width = self.kv_rank
        else:
            out = k.paged_attention(qa, self.num_heads, 1, self.page_dim, self.scale, None, ctx, cache, sinks=self.sinks)
            out_width = self.page_dim
        v = k.headwise_linear(out, self.w_uv, out_width, self.value_dim)
        return k.pending_linear(v, self.w_o)
