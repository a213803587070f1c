"""Feed-forward building blocks shared by the model families.

  * route():       fp32 router with softmax or sigmoid scores, top-k and
                   optional renormalisation of the chosen weights (torch
                   ops; SparseMoE uses the one-kernel ops.moe_route);
  * sparse_moe():  expert dispatch: rows are sorted by expert once (one
                   host read of the per-expert counts per call) and every
                   expert runs the dense GEMM path over its slice, with the
                   routing weight on the expert's output or on its input;
  * GatedMLP / SparseMoE: parameter holders driven by engine.config.MlpSpec,
                   used by the heterogeneous (per-layer spec) models.

The Llama family's Mixtral layers call route()/sparse_moe() too.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from production_stack_amd import ops
from production_stack_amd.engine.config import MlpSpec
from production_stack_amd.ops import gemm_policy


def route(x: torch.Tensor, router_w: torch.Tensor, top: int,
          score: str = "softmax", renormalize: bool = True,
          correction: Optional[torch.Tensor] = None, scale: float = 1.0,
          renorm_eps: float = 0.0):
    """Returns (weights fp32 [T, top], expert ids [T, top]). The logits are
    an fp32 product of the (up-cast) activations and router weights.
    correction (fp32 [experts]): added to the softmax scores for the choice
    only, the weights are the plain scores; the chosen weights are divided
    by (their sum + renorm_eps) when renormalize, then multiplied by
    scale."""
    logits = F.linear(x.float(), router_w.float())
    if score == "softmax":
        probs = torch.softmax(logits, dim=-1)
        if correction is not None:
            _, sel = torch.topk(probs + correction, top, dim=-1)
            weights = probs.gather(-1, sel)
        else:
            weights, sel = torch.topk(probs, top, dim=-1)
    elif score == "sigmoid":
        # rank by the logits: the sigmoid is monotonic but saturates to
        # exactly 1.0 in fp32, which would tie large scores
        _, sel = torch.topk(logits, top, dim=-1)
        weights = torch.sigmoid(logits.gather(-1, sel))
    else:
        raise ValueError(f"unknown router score {score!r}")
    if renormalize:
        weights = weights / (weights.sum(dim=-1, keepdim=True) + renorm_eps)
    if scale != 1.0:
        weights = weights * scale
    return weights, sel


def sparse_moe(x: torch.Tensor, weights: torch.Tensor, sel: torch.Tensor,
               n_experts: int,
               expert_fn: Callable[[int, torch.Tensor], torch.Tensor],
               weight_on_input: bool = False,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sum over chosen experts of  w * expert(x)  (or expert(w * x)).

    expert_fn(e, rows_of_x) -> rows_of_y. `out` (zero-filled [T, width],
    any float dtype) is accumulated into and returned; it defaults to x's
    dtype."""
    T, K = sel.shape
    if out is None:
        out = torch.zeros_like(x)
    flat = sel.reshape(-1)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=n_experts).tolist()
    rows_sorted = torch.div(order, K, rounding_mode="floor")
    w_sorted = weights.reshape(-1)[order]
    start = 0
    for e, n in enumerate(counts):
        if n == 0:
            continue
        rows = rows_sorted[start:start + n]
        w = w_sorted[start:start + n]
        start += n
        xe = x.index_select(0, rows)
        if weight_on_input:
            xe = (xe.float() * w.unsqueeze(-1)).to(x.dtype)
            ye = expert_fn(e, xe)
        elif out.dtype == torch.float32:
            # fp32 accumulator: the fp32 routing weight is applied unrounded
            ye = expert_fn(e, xe).float() * w.unsqueeze(-1)
        else:
            ye = expert_fn(e, xe) * w.to(x.dtype).unsqueeze(-1)
        out.index_add_(0, rows, ye.to(out.dtype))
    return out


class GatedMLP(nn.Module):
    """down(act(gate x) * up x); gate and up are one fused projection. The
    fused in-projection may be run by the caller together with other
    consumers of the same input (see in_params / forward_from_proj).
    gated False: down(act(up x)), `gate_up` then holds the up rows only."""

    def __init__(self, width: int, ff: int, act: str, limit: float,
                 dtype: torch.dtype, gated: bool = True) -> None:
        super().__init__()
        self.ff, self.act, self.limit, self.gated = ff, act, limit, gated
        self.in_rows = (2 if gated else 1) * ff
        self.gate_up = nn.Parameter(
            torch.empty(self.in_rows, width, dtype=dtype))
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype))

    def in_params(self):
        return [self.gate_up]

    def inner(self, proj: torch.Tensor,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """proj [T, 2*ff] = gate | up (or [T, ff] without a gate)  ->
        activation [T, ff]."""
        if not self.gated:
            return ops.gated_act(proj, None, self.act, self.limit, out=out)
        return ops.gated_act(proj[:, :self.ff], proj[:, self.ff:], self.act,
                             self.limit, out=out)

    def forward_from_proj(self, proj: torch.Tensor) -> torch.Tensor:
        return gemm_policy.linear(self.inner(proj), self.down)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward_from_proj(gemm_policy.linear(x, self.gate_up))


class SparseMoE(nn.Module):
    """Routed experts (+ optional always-on shared expert scaled by a
    per-token sigmoid gate), configured by an MlpSpec. The router may have
    `identity` outputs beyond the experts: choosing one of them returns
    the (weighted) input itself."""

    def __init__(self, width: int, spec: MlpSpec, dtype: torch.dtype) -> None:
        super().__init__()
        self.spec = spec
        E, ff = spec.experts, spec.ff
        self.router = nn.Parameter(
            torch.empty(E + spec.identity, width, dtype=dtype))
        self.correction = (
            nn.Parameter(torch.empty(E + spec.identity, dtype=torch.float32))
            if spec.correction else None)
        # without a gate branch the tensor holds the up rows only
        self.experts_gate_up = nn.Parameter(
            torch.empty(E, (2 if spec.gated else 1) * ff, width,
                        dtype=dtype))
        self.experts_down = nn.Parameter(
            torch.empty(E, width, ff, dtype=dtype))
        self.shared = None
        self.shared_gate = None
        if spec.shared_ff:
            self.shared = GatedMLP(width, spec.shared_ff, spec.act,
                                   spec.shared_limit, dtype, spec.gated)
            if spec.shared_gate:
                self.shared_gate = nn.Parameter(
                    torch.empty(1, width, dtype=dtype))
        self._fused_in = None

    def _apply(self, fn, *a, **kw):
        # the fused input weight is a plain tensor rebuilt after a move
        self._fused_in = None
        return super()._apply(fn, *a, **kw)

    def fused_in(self) -> torch.Tensor:
        """The shared expert's gate | up | scalar-gate rows as one weight;
        the parts become views of it."""
        w = self._fused_in
        if w is None:
            parts = self.in_params()
            w = torch.cat([p.data for p in parts], dim=0).contiguous()
            off = 0
            for p in parts:
                p.data = w[off:off + p.shape[0]]
                off += p.shape[0]
            self._fused_in = w
        return w

    def in_params(self):
        """Parameters the caller may fold into a fused projection of the
        layer input: shared gate|up, then the shared expert's scalar
        gate."""
        if self.shared is None:
            return []
        if self.shared_gate is None:
            return [self.shared.gate_up]
        return [self.shared.gate_up, self.shared_gate]

    # decode-sized batches touch (nearly) every expert's weights anyway:
    # up to this many rows all experts run over all rows as three batched
    # GEMMs with the routing weight (0 for experts a row did not choose)
    # folded in, instead of a host-side loop that needs the per-expert row
    # counts on the host every layer
    DENSE_MAX_ROWS = 128

    def _all_experts(self, x: torch.Tensor, wm: torch.Tensor,
                     shared_y: Optional[torch.Tensor] = None,
                     shared_gate: Optional[torch.Tensor] = None
                     ) -> torch.Tensor:
        """Every expert over every row; exact because the experts have no
        biases: a zero-weighted input (or output) contributes exactly 0.
        wm fp32 [T, router outputs]: the routing weights, zero where an
        output was not chosen. With the weight on the experts' outputs, the
        weighted sum, the identity outputs and the gated shared expert
        (shared_y [T, W], shared_gate [T, 1] pre-sigmoid, None = joins
        unscaled) are one kernel."""
        sp = self.spec
        T, E, ff = x.shape[0], sp.experts, sp.ff
        if sp.weight_on_input:
            w_id = (wm[:, E:].sum(dim=1, keepdim=True) if sp.identity
                    else None)
            we = wm[:, :E].t().unsqueeze(-1)            # [E, T, 1]
            xe = (x.float().unsqueeze(0) * we).to(x.dtype)
        else:
            xe = x.unsqueeze(0).expand(E, T, x.shape[1])
        gu = torch.bmm(xe, self.experts_gate_up.transpose(1, 2))
        gu2 = gu.view(E * T, gu.shape[2])
        if sp.gated:
            act = ops.gated_act(gu2[:, :ff], gu2[:, ff:], sp.act, sp.limit)
        else:
            act = ops.gated_act(gu2, None, sp.act, sp.limit, out=gu2)
        y = torch.bmm(act.view(E, T, ff), self.experts_down.transpose(1, 2))
        if not sp.weight_on_input:
            return ops.moe_combine(y, wm, x, E, shared_y, shared_gate)
        y = y.float().sum(dim=0)
        if w_id is not None:
            y += x.float() * w_id
        if shared_y is not None:
            y += (shared_y.float() * torch.sigmoid(shared_gate.float())
                  if shared_gate is not None else shared_y.float())
        return y

    def _expert(self, e: int, xe: torch.Tensor) -> torch.Tensor:
        if e >= self.spec.experts:      # identity expert
            return xe
        ff = self.spec.ff
        gu = gemm_policy.linear(xe, self.experts_gate_up[e])
        if self.spec.gated:
            act = ops.gated_act(gu[:, :ff], gu[:, ff:], self.spec.act,
                                self.spec.limit)
        else:
            act = ops.gated_act(gu, None, self.spec.act, self.spec.limit,
                                out=gu)
        return gemm_policy.linear(act, self.experts_down[e])

    def forward_from_proj(self, x: torch.Tensor,
                          proj: Optional[torch.Tensor],
                          dense: Optional[bool] = None) -> torch.Tensor:
        """x: layer input [T, width]; proj: the shared expert's fused
        projection [T, shared in-rows (+ 1 with a scalar gate)] (None
        without a shared expert).
        dense=True insists on the all-experts path (no host read: what a
        captured decode step needs), None picks by batch size. Returns fp32
        [T, width]: several experts' outputs are summed in fp32."""
        sp = self.spec
        # one kernel: logits, scores, choice, weights, dense weight matrix
        weights, sel, wm = ops.moe_route(
            x, self.router, sp.top, sp.score, sp.renormalize,
            self.correction, sp.route_scale, sp.renorm_eps)
        T = x.shape[0]
        y = gate = None
        if self.shared is not None:
            rows = self.shared.in_rows
            y = self.shared.forward_from_proj(proj[:, :rows])
            if self.shared_gate is not None:
                gate = proj[:, rows:]
        if dense is None:
            dense = T <= self.DENSE_MAX_ROWS and T * sp.top >= sp.experts
        if dense:
            return self._all_experts(x, wm, y, gate)
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        sparse_moe(x, weights, sel, sp.experts + sp.identity, self._expert,
                   weight_on_input=sp.weight_on_input, out=out)
        if y is not None:
            out += (y.float() * torch.sigmoid(gate.float())
                    if gate is not None else y.float())
        return out

    def forward(self, x: torch.Tensor,
                dense: Optional[bool] = None) -> torch.Tensor:
        proj = (gemm_policy.linear(x, self.fused_in())
                if self.shared is not None else None)
        return self.forward_from_proj(x, proj, dense)
