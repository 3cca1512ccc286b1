"""Attention over one cached latent vector per token."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.spec import PagedKVSpec
from ..kernels.limits import MAX_LATENT_ROW, check_attention_sizes
from .base import Mixer, Part, PositionEncoding
from .context import MixerPlan, PlanInput, StepContext
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Causal attention whose keys and values are linear maps of a latent c_t of `kv_rank` numbers
    per token, beside one rotated key part r_t of `rot_dim` numbers that all heads share.

    With h the mixer's input:  [c'_t ; r'_t] = Wdkv h_t,  c_t = rmsnorm(c'_t) * w (32-bit),
    r_t = rotate(r'_t, t);  per head i: q_i = [u_i ; rotate(p_i, t)] (rows of Wq, `dim` unrotated
    then `rot_dim` rotated), key k_i,j = [Wuk_i c_j ; r_j], value v_i,j = Wuv_i c_j,
    score s_i,tj = (u_i . Wuk_i c_j + p_i . r_j) * scale for j <= t,
    weights a = exp(s) / (sum_j exp(s) + exp(sink_i)) (the sink is a learned number per head: a
    term of the denominator without key or value), out = Wo [gate_i * sum_j a_ij v_ij]_i with
    gate = sigmoid(Wg h) (one number per head and token).

    Only c and r are cached, and the products with Wuk and Wuv are taken out of the sum over the
    keys:  u_i . Wuk_i c_j = (Wuk_i^T u_i) . c_j  and  sum_j a_ij Wuv_i c_j = Wuv_i (sum_j a_ij c_j).
    So every head's query becomes a vector of kv_rank + rot_dim numbers, all heads attend over the
    SAME cached rows [c_j ; r_j] with the values c_j (attention with one key/value head, the heads
    side by side in the matrix cores' columns), and Wuv is applied once per token to the attended
    latent.  The pages hold c twice: as part of the key row and, transposed, as the value.

    q_rank: the queries go through a latent of their own: c_q = rmsnorm(Wdq h) * w_q (32-bit), q = Wuq c_q.  The
    input product then has Wdq's rows in a product of its own, whose normed result feeds the query product.

    A rotation that pairs neighbouring dims (`interleaved`) is served by reordering, once, the rows that make
    the rotated parts of queries and key (a dot product does not care in which order both list their dims).

    kv_source: True for a site that reads an earlier site's cache (`OrderEntry.reads_cache_of`): it
    has no Wdkv and writes nothing; its cache spec equals the owner's.
    """

    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        rot_dim: int,
        value_dim: int,
        kv_rank: int,
        scale: float,
        norm_eps: float,
        position: Optional[PartSpec] = None,
        reads_cache: bool = False,
        sink: bool = True,
        output_gate: bool = True,
        q_rank: Optional[int] = None,
    ) -> None:
        if min(hidden_size, num_heads, head_dim, rot_dim, value_dim, kv_rank) <= 0:
            raise ValueError("LatentAttention sizes must be > 0")
        if not scale > 0:
            raise ValueError("scale must be > 0")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.rot_dim = int(rot_dim)
        self.value_dim = int(value_dim)
        self.kv_rank = int(kv_rank)
        self.scale = float(scale)
        self.norm_eps = float(norm_eps)
        self.reads_cache = bool(reads_cache)
        self.has_sink = bool(sink)
        self.output_gate = bool(output_gate)
        if q_rank is not None and q_rank <= 0:
            raise ValueError("q_rank must be > 0 or None")
        self.q_rank = None if q_rank is None else int(q_rank)
        # the one head size that the attention kernels and the pages see: a cached row [c ; r], padded
        self.kernel_dim = -(-(self.kv_rank + self.rot_dim) // 16) * 16
        # rows of up to 256 run on the matrix cores (in bfloat16); wider ones, up to 1,024, the plain kernel
        check_attention_sizes(num_heads, 1, self.kernel_dim, limit=MAX_LATENT_ROW)
        self.position: Optional[PositionEncoding] = build_part("position", position) if position is not None else None
        if self.position is not None and getattr(self.position, "rotary_dim", self.rot_dim) > self.rot_dim:
            raise ValueError("the rotation covers more dimensions than the rotated part has")
        self.in_weight: Optional[torch.Tensor] = None
        self.latent_norm_weight: Optional[torch.Tensor] = None
        self.uk_weight: Optional[torch.Tensor] = None
        self.uv_weight: Optional[torch.Tensor] = None
        self.sink: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.dq_weight: Optional[torch.Tensor] = None
        self.q_norm_weight: Optional[torch.Tensor] = None
        self.uq_weight: Optional[torch.Tensor] = None

    # rows of the one input product: queries, then (unless the cache is another site's) latent and
    # rotated key part, then the gate
    @property
    def q_rows(self) -> int:
        return self.num_heads * (self.head_dim + self.rot_dim)

    @property
    def kv_rows(self) -> int:
        return 0 if self.reads_cache else self.kv_rank + self.rot_dim

    @property
    def gate_rows(self) -> int:
        return self.num_heads if self.output_gate else 0

    def param_specs(self) -> dict[str, ParamSpec]:
        own_q = 0 if self.q_rank is not None else self.q_rows
        specs = {
            "in_weight": ParamSpec((own_q + self.kv_rows + self.gate_rows, self.hidden_size)),
            "uk_weight": ParamSpec((self.num_heads * self.head_dim, self.kv_rank)),
            "uv_weight": ParamSpec((self.num_heads * self.value_dim, self.kv_rank)),
            "o_weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim)),
        }
        if not self.reads_cache:
            specs["latent_norm_weight"] = ParamSpec((self.kv_rank,), init="one_plus_normal", keep_stored_precision=True)
        if self.has_sink:
            specs["sink"] = ParamSpec((self.num_heads,), keep_stored_precision=True)
        if self.q_rank is not None:
            specs["dq_weight"] = ParamSpec((self.q_rank, self.hidden_size))
            specs["q_norm_weight"] = ParamSpec((self.q_rank,), init="one_plus_normal", keep_stored_precision=True)
            specs["uq_weight"] = ParamSpec((self.q_rows, self.q_rank))
        if self.q_rank is not None and self.kv_rows + self.gate_rows == 0:
            del specs["in_weight"]  # a site that reads another's cache, ungated: nothing but queries to project
        return specs

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        # Wuk per head transposed, [head, kv_rank, dim]: the query of a head goes through it as
        # through any weight stored [out, in]
        uk = self.uk_weight.view(self.num_heads, self.head_dim, self.kv_rank)
        self.uk_t = uk.transpose(1, 2).contiguous()
        self.uv = self.uv_weight.view(self.num_heads, self.value_dim, self.kv_rank)
        if self.sink is not None:
            self.sink = self.sink.to(torch.float32)
        order = self.position.half_split_order() if self.position is not None else None
        if order is not None and order != list(range(len(order))):
            # neighbouring pairs -> halves: the rows of every head's rotated query part, and of the key part
            index = torch.tensor(order, device=device)
            qd = self.head_dim + self.rot_dim
            q_matrix = self.uq_weight if self.q_rank is not None else self.in_weight
            for head in range(self.num_heads):
                at = head * qd + self.head_dim
                q_matrix[at : at + self.rot_dim] = q_matrix[at : at + self.rot_dim][index]
            if not self.reads_cache:
                at = (0 if self.q_rank is not None else self.q_rows) + self.kv_rank
                self.in_weight[at : at + self.rot_dim] = self.in_weight[at : at + self.rot_dim][index]

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(1, self.kernel_dim)

    def plan(self, ops, shape: PlanInput) -> Optional[MixerPlan]:
        make = getattr(ops, "attention_plan", None)
        return make(shape) if make is not None else None

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        cache = ctx.kv(site)
        if cache.writable == self.reads_cache:
            raise RuntimeError("a latent-attention site owns its cache exactly when it has a down-projection of its own")
        rotation = self.position.rotation(ctx) if self.position is not None else None
        # the input product's sums stay 32-bit: the latent's norm, the rotation and the gate read them unrounded
        queries = None
        if self.q_rank is not None:
            latent = ops.rmsnorm(
                ops.linear(h, self.dq_weight, None, out_dtype=torch.float32), self.q_norm_weight, self.norm_eps
            )
            queries = ops.linear(latent, self.uq_weight, None, out_dtype=torch.float32)
        if self.in_weight is not None:
            projected = ops.linear(h, self.in_weight, None, out_dtype=torch.float32)
        else:
            projected = queries
        q_plain, q_latent, gate = ops.latent_prepare(
            projected,
            heads=self.num_heads,
            head_dim=self.head_dim,
            rot_dim=self.rot_dim,
            kv_rank=self.kv_rank,
            own_cache=not self.reads_cache,
            gated=self.output_gate,
            norm_weight=self.latent_norm_weight,
            eps=self.norm_eps,
            rotation=rotation,
            slot_mapping=cache.slot_mapping,
            key_pages=cache.key,
            value_pages=cache.value,
            block_size=cache.block_size,
            kernel_dim=self.kernel_dim,
            **({"queries": queries} if queries is not None else {}),
        )
        if cache.writable:
            cache.written()
        # every head's unrotated query through its Wuk^T, into the leading kv_rank columns of its latent query
        ops.heads_linear(q_plain, self.uk_t, in_stride=self.head_dim, out=q_latent, out_stride=self.kernel_dim)
        cache.reading()
        attended = ops.paged_attention(
            q_latent,
            cache.key,
            cache.value,
            cache.block_table,
            ctx,
            num_heads=self.num_heads,
            num_kv_heads=1,
            head_dim=self.kernel_dim,
            block_size=cache.block_size,
            scale=self.scale,
            window=None,
            plan=ctx.plan(getattr(ops, "ATTENTION_PLAN", None)),
            **({"sinks": self.sink} if self.sink is not None else {}),
        )
        # the attended latent of every head through its Wuv, times the head's gate
        merged = ops.heads_linear(
            attended, self.uv, in_stride=self.kernel_dim, **({"row_scale": gate} if gate is not None else {})
        )
        return ops.linear(merged, self.o_weight, None, for_stream=True)
