"""Sparse mixture of experts with an optional gated shared expert.

Per token (ferrox-models/src/decoder.rs:2895-2924, 2567-2682): router logits
r = W_r x; a gating function over all experts and the k best of them
(ferrox-moe/src/lib.rs:333-355); each chosen expert is a gated feed-forward
(lib.rs:655-658); their outputs are summed with the routing weights in selection
order (lib.rs:735-745); a shared expert, scaled by sigmoid(w_g . x), is added
(decoder.rs:2660-2679).
"""
from __future__ import annotations

import torch

from .. import debug, limits, ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec
from .linear import matmul, same_dtype
from .mlp import GatedMLP

GATINGS = {"softmax": ops.GATE_SOFTMAX, "sigmoid": ops.GATE_SIGMOID}
FRONT_MAX_TOKENS = 128       # up to so many tokens the norm, the router, the selection and the sort are one launch (the
                             # kernel takes 256; from 192 on its blocks, which all read the router's rows, fall behind)
PIECES_MAX_PAIRS = 1024      # up to so many (token, slot) pairs the shared expert's pieces run as experts that every token takes
                             # (measured at both models' sizes: ahead up to here, behind from 1,536 pairs on)
OVERLAP_MAX_TOKENS = 8192    # up to here the shared expert runs beside the routed ones on a second stream
_side_streams: dict = {}


def side_stream(device) -> torch.cuda.Stream:
    """One extra stream per device, of the default priority."""
    key = torch.device(device)
    if key not in _side_streams:
        _side_streams[key] = torch.cuda.Stream(device=key)
    return _side_streams[key]


@FEED_FORWARDS.register("sparse_moe")
class SparseMoE(FeedForward):
    kernel_libraries = ("elementwise", "gemm", "moe")
    norms_after = True   # forward(..., then_norm=norm) may leave norm(residual) in ctx.carry for the next layer

    def __init__(self, hidden_size: int, n_experts: int, top_k: int, expert_intermediate_size: int,
                 norm_topk_prob: bool, gating: str = "softmax", shared_intermediate_size: int = 0,
                 shared_gate: bool = True, activation: str = "silu"):
        if not 1 <= top_k <= n_experts:
            raise ValueError(f"top_k {top_k} must lie in 1..{n_experts}")
        if n_experts > limits.MOE_MAX_EXPERTS or top_k > limits.MOE_MAX_TOP_K:
            raise ValueError(f"{n_experts} experts / top_k {top_k}: the routing kernels take up to "
                             f"{limits.MOE_MAX_EXPERTS} experts and {limits.MOE_MAX_TOP_K} per token")
        if gating not in GATINGS:
            raise ValueError(f"gating '{gating}' is not one of {sorted(GATINGS)}")
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {sorted(ops.ACTIVATIONS)}")
        self.activation = activation
        self.hidden_size, self.n_experts, self.top_k = int(hidden_size), int(n_experts), int(top_k)
        self.expert_intermediate_size = int(expert_intermediate_size)
        self.norm_topk_prob, self.gating = bool(norm_topk_prob), GATINGS[gating]
        self.shared = GatedMLP(hidden_size, shared_intermediate_size, activation) if shared_intermediate_size > 0 else None
        self.has_shared_gate = bool(shared_gate) and self.shared is not None
        self.router = self.w_gate_up = self.w_down = None

    def children(self):
        return [("shared_expert.", self.shared)] if self.shared is not None else []

    def param_specs(self):
        H, I = self.hidden_size, self.expert_intermediate_size
        specs = {"gate.weight": ParamSpec((self.n_experts, H))}
        for e in range(self.n_experts):
            specs[f"experts.{e}.gate_proj.weight"] = ParamSpec((I, H))
            specs[f"experts.{e}.up_proj.weight"] = ParamSpec((I, H))
            specs[f"experts.{e}.down_proj.weight"] = ParamSpec((H, I))
        if self.has_shared_gate:
            specs["shared_expert_gate.weight"] = ParamSpec((1, H))
        return specs

    def load(self, fetch):
        router = fetch("gate.weight")
        gu, dn = [], []
        for e in range(self.n_experts):
            gu.append(torch.cat(same_dtype([fetch(f"experts.{e}.gate_proj.weight"),
                                            fetch(f"experts.{e}.up_proj.weight")]), dim=0))
            dn.append(fetch(f"experts.{e}.down_proj.weight"))
        # A shared expert whose width is a multiple of the experts' is also kept cut into pieces of their
        # shape, after the experts in the same tensors: for few tokens it then runs as experts that every
        # token takes, inside the experts' two launches (its own copy serves many tokens).
        I, E, H = self.expert_intermediate_size, self.n_experts, self.hidden_size
        self.shared_pieces = 0
        if self.shared is not None and self.shared.intermediate_size % I == 0:
            sg, su, sdn = (fetch("shared_expert." + n) for n in ("gate_proj.weight", "up_proj.weight", "down_proj.weight"))
            if all(t.dtype == gu[0].dtype for t in gu + dn + [sg, su, sdn]):
                S = self.shared.intermediate_size // I
                for s in range(S):
                    gu.append(torch.cat([sg[s * I:(s + 1) * I], su[s * I:(s + 1) * I]], dim=0))
                    dn.append(sdn[:, s * I:(s + 1) * I])
                self.shared_pieces = S
            del sg, su, sdn
        all_gu = torch.stack(same_dtype(gu)).contiguous()             # [E (+S), 2*I, H]
        all_dn = torch.stack(same_dtype(dn)).contiguous()             # [E (+S), H, I]
        del gu, dn
        # streamed weights are kept in slabs of 64 k where the kernels take that
        self.kblocked = all_gu.dtype == torch.bfloat16 and all_dn.dtype == torch.bfloat16 and H % 64 == 0 and I % 64 == 0
        if self.kblocked:
            all_gu, all_dn = ops.to_kblocked(all_gu), ops.to_kblocked(all_dn)
        self.w_gate_up_all, self.w_down_all = all_gu, all_dn
        self.w_gate_up, self.w_down = all_gu[:E], all_dn[:E]
        if self.has_shared_gate:     # the gate's row rides along as column E of the router product
            router = torch.cat(same_dtype([router, fetch("shared_expert_gate.weight").reshape(1, -1)]), dim=0)
        self.router = router.contiguous()

    @staticmethod
    def _then(then_norm, ctx, n_tokens) -> dict:
        """How the combine prepares the new rows for the next block's norm: `then_norm` is (norm, whether the
        block takes an ops.ScaleLater).  For up to 64 rows (what the product for few rows takes) the combine also
        writes them times the norm's weight, with sums of squares, and the product that follows applies the
        scale: the norm costs no launch.  (For many rows a norm kernel of its own is as fast.)"""
        if then_norm is None or then_norm[0].rms_params() is None:
            return {}
        norm, later_ok = then_norm
        if n_tokens <= 64 and later_ok and ctx.act_dtype == torch.bfloat16:
            return dict(scale_later=(*norm.rms_params(), ctx.act_dtype))
        return {}

    def forward_from_residual(self, norm, ctx, residual, then_norm=None) -> bool:
        """Few tokens: the norm and the router are one launch; up to 16 tokens the expert products group the
        (token, slot) pairs themselves instead of reading a sorted layout, for more that launch also sorts them."""
        T = residual.shape[0]
        rms = norm.rms_params()
        if T > FRONT_MAX_TOKENS or ctx.act_dtype != torch.bfloat16 or rms is None:
            return False
        if T > 64 and not (self.shared_pieces and T * self.top_k <= PIECES_MAX_PAIRS and self.kblocked
                           and ctx.act_dtype == self.w_gate_up_all.dtype):
            return False        # (more than 64 tokens: only where the shared expert's pieces ride along, see forward)
        debug.region("router")
        rows_ok = self.hidden_size % 8 == 0 and self.expert_intermediate_size % 8 == 0
        unsorted = T <= 16 and T * self.top_k <= 64 and rows_ok       # the expert products take the pairs unsorted
        # otherwise the shared expert's pieces ride along as experts that every token takes, behind the sorted
        # pairs, and the launch that selects the experts also sorts the pairs by expert
        S = self.shared_pieces if ctx.act_dtype == self.w_gate_up_all.dtype and T * self.top_k <= 2048 else 0
        front = ops.moe_front(residual, rms[0], rms[1], self.router, self.n_experts, self.top_k,
                              self.norm_topk_prob, self.gating, self.has_shared_gate, align=None if unsorted else S)
        if front is None:
            return False
        x, ids, weights, gate, sort = front
        if unsorted:
            self.forward(x, ctx, residual, routed=(ids, weights, gate, None, None, None, None), then_norm=then_norm)
        else:
            if sort is None:
                sort = ops.moe_align(ids, self.n_experts, always=S)
            self.forward(x, ctx, residual, routed=(ids, weights, gate) + sort, then_norm=then_norm, sorted_pieces=S)
        return True

    def forward(self, x, ctx, residual, routed=None, then_norm=None, sorted_pieces: int = 0) -> None:
        T = x.shape[0]
        then = self._then(then_norm, ctx, T)
        if sorted_pieces:
            # up to 64 tokens, sorted pairs: the shared expert as `sorted_pieces` pieces behind the experts in the same
            # two launches (its own two products would stream its weights to 64 rows far below the memory's speed)
            ids, weights, gate, offsets, sorted_token, sorted_pair, _ = routed
            if debug.routing_trace is not None:
                debug.routing_trace.put(ids)
            S, n = sorted_pieces, ids.numel()
            kb = dict(w_kblocked=True) if self.kblocked else {}
            debug.region("experts gate/up")
            act = matmul(x, self.w_gate_up_all, epilogue=ops.EPI_GATED, activation=self.activation, a_rows=sorted_token, expert_offsets=offsets,
                         n_rows=n + S * T, **kb)
            debug.region("experts down")
            y = matmul(act, self.w_down_all, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair, **kb)
            debug.region("combine")
            ctx.carry = ops.moe_combine(residual, y[:n], None, weights, self.top_k, shared=y[n:].view(S, T, -1), gate=gate,
                                        **then)
            return
        if routed is not None and routed[3] is None and self.shared_pieces and x.dtype == self.w_gate_up_all.dtype:
            # few tokens, unsorted pairs, shared expert as pieces: two launches do all experts
            ids, weights, gate = routed[:3]
            if debug.routing_trace is not None:
                debug.routing_trace.put(ids)
            S, n = self.shared_pieces, ids.numel()
            debug.region("experts gate/up")
            act = ops.gemm(x, self.w_gate_up_all, epilogue=ops.EPI_GATED, activation=self.activation, pair_ids=ids, pair_div=self.top_k,
                           always=(S, T, True), w_kblocked=self.kblocked)
            debug.region("experts down")
            y = ops.gemm(act, self.w_down_all, epilogue=ops.EPI_STORE_F32, pair_ids=ids, always=(S, T, False),
                         w_kblocked=self.kblocked)
            debug.region("combine")
            ctx.carry = ops.moe_combine(residual, y[:n], None, weights, self.top_k, shared=y[n:].view(S, T, -1), gate=gate, **then)
            return
        if (routed is None and self.shared_pieces and 64 < T and T * self.top_k <= PIECES_MAX_PAIRS and self.kblocked
                and x.dtype == self.w_gate_up_all.dtype):
            # A step of a few hundred tokens: the shared expert's pieces ride along behind the sorted pairs as they
            # do for up to 64 tokens.  Its own two products would run on tiles too few for the GPU (its down
            # product's 2,048 weight rows give 16 tiles of 128 columns) beside launches that the host cannot
            # issue faster than the GPU runs them.
            debug.region("router")
            if self.router.shape[0] <= 64 and self.router.dtype == x.dtype:      # (as below: the router's rows as the short side)
                logits = ops.gemm(self.router, x, epilogue=ops.EPI_STORE_F32).t()
            else:
                logits = matmul(x, self.router, epilogue=ops.EPI_STORE_F32)
            ids, weights, gate = ops.router_select(logits, self.n_experts, self.top_k, self.norm_topk_prob, self.gating,
                                                   self.has_shared_gate)
            S = self.shared_pieces
            self.forward(x, ctx, residual, routed=(ids, weights, gate) + ops.moe_align(ids, self.n_experts, always=S),
                         then_norm=then_norm, sorted_pieces=S)
            return
        overlap = self.shared is not None and T <= OVERLAP_MAX_TOKENS
        if overlap:
            # the shared expert runs on a second stream beside the router and the routed experts, and its output
            # joins in the combine: with few tokens both halves wait for weights from memory, with many the
            # blocks of one fill the CUs that the last round of the other's tiles leaves idle
            main, side = torch.cuda.current_stream(), side_stream(x.device)
            fork, join = torch.cuda.Event(), torch.cuda.Event()
            fork.record(main)
            side.wait_event(fork)
            with torch.cuda.stream(side):
                debug.region("shared expert")
                shared_out = self.shared.output(x)
                join.record(side)
        if routed is None:
            debug.region("router")
            if T > 64 and self.router.shape[0] <= 64 and self.router.dtype == x.dtype:
                # few experts, many tokens: the router's rows are the short side of the product, so the
                # kernel for few rows streams the activations once; the logits come out transposed
                logits = ops.gemm(self.router, x, epilogue=ops.EPI_STORE_F32).t()
            else:
                logits = matmul(x, self.router, epilogue=ops.EPI_STORE_F32)
            routed = ops.route(logits, self.n_experts, self.top_k, self.norm_topk_prob, self.gating,
                               self.has_shared_gate)
        ids, weights, gate, offsets, sorted_token, sorted_pair, _ = routed
        if debug.routing_trace is not None:
            debug.routing_trace.put(ids)
        kb = dict(w_kblocked=True) if self.kblocked else {}
        debug.region("experts gate/up")
        if offsets is None:      # few pairs, unsorted: row p of `act` and of `y` is pair p
            act = ops.gemm(x, self.w_gate_up, epilogue=ops.EPI_GATED, activation=self.activation, pair_ids=ids, pair_div=self.top_k, **kb)
            debug.region("experts down")
            y = ops.gemm(act, self.w_down, epilogue=ops.EPI_STORE_F32, pair_ids=ids, **kb)
        else:
            act = matmul(x, self.w_gate_up, epilogue=ops.EPI_GATED, activation=self.activation, a_rows=sorted_token,
                         expert_offsets=offsets, n_rows=T * self.top_k, **kb)
            debug.region("experts down")
            # each expert's rows go back to the place of their (token, slot) pair
            y = matmul(act, self.w_down, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair, **kb)
        debug.region("combine")
        if overlap:
            main.wait_event(join)
            shared_out.record_stream(main)
            ctx.carry = ops.moe_combine(residual, y, None, weights, self.top_k, shared=shared_out, gate=gate, **then)
        elif self.shared is None:
            ctx.carry = ops.moe_combine(residual, y, None, weights, self.top_k, **then)
        else:
            ops.moe_combine(residual, y, None, weights, self.top_k)
            self.shared.forward(x, ctx, residual, row_scale=gate)
