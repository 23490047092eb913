"""Dense feed-forward with a gated SiLU."""
import torch

from ..kernels import ops
from ..kernels.tuning import TUNING
from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear, gated_linear, gated_plan, linear_into_norm
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), no biases (ginfer/core/layer/transformer/feedforward.cc:22-25); gate and
    up are one product over the stacked weights, which equals the two separate ones."""

    capturable = True
    takes_scaled_rows = True
    folds_norm = True

    def __init__(self, hidden_size, intermediate_size, dtype, device):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.dtype, self.device = dtype, device
        self.w_gate_up = self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": WeightSpec((I, H)), "up_proj.weight": WeightSpec((I, H)),
                "down_proj.weight": WeightSpec((H, I))}

    def bind_weights(self, t):
        self.w_gate_up = torch.cat([t["gate_proj.weight"], t["up_proj.weight"]], dim=0).contiguous()
        self.w_down = t["down_proj.weight"]

    def kernel_modules(self):
        return ["activation", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, into_norm=None):
        """into_norm = (residual, norm): where the down projection's kernel can, the result is added to the
        residual here and the rows of `norm` come back as ops.ScaledRows."""
        act = gated_linear(x, self.w_gate_up)
        if into_norm is not None:
            folded = linear_into_norm(act, self.w_down, None, *into_norm)
            if folded is not None:
                return folded
        # the result may be partial sums of a K-split product: the norm that follows adds them up
        return linear(act, self.w_down, parts_ok=True)


@register_feed_forward("clamped_glu")
class ClampedGLU(Part):
    """down(g * sigmoid(alpha g) * (u + shift)) with g = min(gate(x), limit) and u = clamp(up(x), -limit, limit); no
    biases.  limit, alpha and shift are the model's constants.  Gate and up are one product over the stacked weights.
    The tensors are named gate, up and down."""

    capturable = True

    def __init__(self, hidden_size, intermediate_size, limit, dtype, device, alpha=1.702, shift=1.0):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        self.dtype, self.device = dtype, device
        self.w_gate_up = self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def bind_weights(self, t):
        self.w_gate_up = torch.cat([t["gate"], t["up"]], dim=0).contiguous()
        self.w_down = t["down"]

    def kernel_modules(self):
        return ["activation", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x):
        # few rows (decode): the weight-streaming product with the activation in its epilogue, where the rules would
        # take that kernel for the SiLU gate too; else the product and the activation's own pass
        if (x.dtype == torch.bfloat16 and ops.gemm_skinny_supported(x, self.w_gate_up)
                and gated_plan(x.shape[0], self.w_gate_up.shape[0], True, False) == ("skinny",)):
            act = ops.gemm_skinny(x, self.w_gate_up, gated=True, gate_bounds=(self.limit, self.alpha, self.shift))
        else:
            act = ops.clamped_glu(linear(x, self.w_gate_up), self.limit, self.alpha, self.shift)
        return linear(act, self.w_down)


@register_feed_forward("squared_relu")
class SquaredReLU(Part):
    """down(relu(up(x))^2): no gate, no biases.  The tensors are named up and down."""

    capturable = True

    def __init__(self, hidden_size, intermediate_size, dtype, device):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.dtype, self.device = dtype, device
        self.w_up = self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def bind_weights(self, t):
        self.w_up, self.w_down = t["up"], t["down"]

    def kernel_modules(self):
        return ["activation", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x):
        # the result may be partial sums of a K-split product: the norm that follows adds them up
        return linear(ops.relu_square(linear(x, self.w_up)), self.w_down, parts_ok=True)


@register_feed_forward("routed_glu")
class RoutedGLU(Part):
    """A mixture of gated feed-forwards.  Router scores z = Wr x + b in 32-bit; every token uses the `top_k` experts with
    the largest scores, weighted by the softmax over those scores alone; an optional shared expert of its own width
    runs for every token and is added.  Expert: down(silu(gate(x)) * up(x)), no biases.

    Two ways, by the number of rows (`TUNING.routed_by_expert_from_rows`; the second way is switched off there for now).  Few rows, and every step that is recorded:
    the experts lie side by side, ONE product gives the gates and ups of all experts (and of the shared one), the
    activation multiplies each expert's columns by the token's weight for it (zero where the token does not use it), and
    ONE product with the down matrices laid side by side adds the experts' results up, in 32-bit.  Many rows (bfloat16):
    the token-expert pairs are grouped by expert, the groups laid side by side as long as the longest, two batched
    products run every expert over its own rows, and a last kernel adds a token's results with their weights; this way
    reads the groups' sizes on the host, so it is never recorded.  Routing is a
    pure function of the token's row, so a token's result does not depend on the batch beyond rounding; in 32-bit
    only the first way runs, and not at all.
    Tensors: router, router.b, e<i>.gate / .up / .down, shared.gate / .up / .down."""

    capturable = True                # the steps that the runner records are short enough for the first way

    def __init__(self, hidden_size, num_experts, top_k, expert_size, dtype, device, shared_size=None, router_bias=True,
                 scoring="softmax_chosen", correction=False, groups=1, keep_groups=1, group_top=2, weight_scale=1.0,
                 weight_floor=0.0):
        """scoring "softmax_chosen": as the class's text.  scoring "sigmoid": scores s = sigmoid(z); the choice goes by s +
        `correction` (a tensor of that name, where correction is set) among the experts of the `keep_groups` best of `groups`
        equal groups of neighbouring experts (a group's score: the sum of its `group_top` largest choice scores); the weights
        are the chosen experts' s divided by their sum + weight_floor, times weight_scale."""
        if scoring not in ("softmax_chosen", "sigmoid"):
            raise ValueError("unknown scoring %r (known: softmax_chosen, sigmoid)" % (scoring,))
        self.scoring, self.correction = scoring, bool(correction)
        self.groups, self.keep_groups, self.group_top = int(groups), int(keep_groups), int(group_top)
        self.weight_scale, self.weight_floor = float(weight_scale), float(weight_floor)
        if scoring == "sigmoid":
            E = int(num_experts)
            if self.groups < 1 or E % self.groups or not 1 <= self.keep_groups <= self.groups \
                    or int(top_k) > self.keep_groups * (E // self.groups) or not 1 <= self.group_top <= 4:
                raise ValueError("%d experts in %d groups of which %d are kept cannot give %d choices"
                                 % (E, self.groups, self.keep_groups, int(top_k)))
        elif correction or self.groups != 1:
            raise ValueError("a correction of the choice and groups of experts belong to the sigmoid scoring")
        self.hidden_size, self.num_experts, self.top_k = int(hidden_size), int(num_experts), int(top_k)
        self.expert_size = int(expert_size)
        self.shared_size = int(shared_size) if shared_size else 0
        self.router_bias = bool(router_bias)
        if not 1 <= self.top_k <= self.num_experts <= ops.ROUTE_MAX_EXPERTS:
            raise ValueError("routing takes 1 <= top_k <= experts <= %d, got top_k %d of %d experts"
                             % (ops.ROUTE_MAX_EXPERTS, self.top_k, self.num_experts))
        self.dtype, self.device = dtype, device
        self.w_router = self.b_router = self.w_gate_up = self.w_down = self.w_correction = None

    def weight_specs(self):
        H, F, S = self.hidden_size, self.expert_size, self.shared_size
        specs = {"router": WeightSpec((self.num_experts, H), std=0.2, keep_32bit=True)}
        if self.router_bias:
            specs["router.b"] = WeightSpec((self.num_experts,), std=0.2, keep_32bit=True)
        if self.correction:
            specs["correction"] = WeightSpec((self.num_experts,), std=0.2, keep_32bit=True)
        for e in range(self.num_experts):
            specs.update({"e%d.gate" % e: WeightSpec((F, H)), "e%d.up" % e: WeightSpec((F, H)),
                          "e%d.down" % e: WeightSpec((H, F))})
        if S:
            specs.update({"shared.gate": WeightSpec((S, H)), "shared.up": WeightSpec((S, H)), "shared.down": WeightSpec((H, S))})
        return specs

    def bind_weights(self, t):
        self.w_router = t["router"].float().contiguous()
        self.b_router = t["router.b"].float().contiguous() if self.router_bias else None
        self.w_correction = t["correction"].float().contiguous() if self.correction else None
        names = ["e%d" % e for e in range(self.num_experts)] + (["shared"] if self.shared_size else [])
        # every expert's gate rows, then its up rows: one expert's share of the stacked matrix is one piece
        self.w_gate_up = torch.cat([t[n + kind] for n in names for kind in (".gate", ".up")], dim=0).contiguous()
        self.w_down = torch.cat([t[n + ".down"] for n in names], dim=1).contiguous()

    def kernel_modules(self):
        return ["routing", "activation", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def route(self, x):
        """(ids int32 [T, top_k], weights float32 [T, top_k], the weights as rows over all experts [T, E])."""
        z = ops.router_scores(x, self.w_router, self.b_router)
        if self.scoring == "sigmoid":
            return ops.route_sigmoid_groups(z, self.top_k, self.w_correction, self.groups, self.keep_groups, self.group_top,
                                            True, self.weight_floor, self.weight_scale)
        return ops.route_topk(z, self.top_k)

    def forward(self, x):
        ids, weights, dense = self.route(x)
        if x.dtype == torch.bfloat16 and x.shape[0] >= TUNING.routed_by_expert_from_rows:
            if not TUNING.routed_by_expert_allowed:
                raise RuntimeError("the experts as a batched product over their own rows: switched off (an unexplained "
                                   "memory fault at large sizes); see kernels/tuning.py")
            return self._by_expert(x, ids, weights)
        act = ops.weighted_silu_mul(linear(x, self.w_gate_up), dense, self.expert_size)
        return linear(act, self.w_down, parts_ok=True)     # maybe partial sums: the norm that follows adds them up

    def _by_expert(self, x, ids, weights):
        E, F, S, H = self.num_experts, self.expert_size, self.shared_size, self.hidden_size
        offsets, pair_of_row, row_of_pair = ops.route_sort(ids, E)
        bounds = offsets.tolist()                    # the host waits here for the groups' sizes
        # every expert's group as long as the longest, so that the experts are the batch of two batched products
        capacity = -(-max(max(b - a for a, b in zip(bounds, bounds[1:])), 1) // 16) * 16
        rows = ops.gather_pair_rows(x, pair_of_row, ids, offsets, capacity)
        gate_up = torch.bmm(rows, self.w_gate_up[:2 * F * E].view(E, 2 * F, H).transpose(1, 2))
        act = ops.silu_mul(gate_up.view(E * capacity, 2 * F))
        down = self.w_down.as_strided((E, H, F), (F, self.w_down.stride(0), 1))       # expert e: the columns [eF, (e+1)F)
        y = torch.bmm(act.view(E, capacity, F), down.transpose(1, 2))
        shared = None
        if S:
            shared = torch.mm(gated_linear(x, self.w_gate_up[2 * F * E:]), self.w_down[:, F * E:].t())
        return ops.combine_pairs(y, shared, weights, row_of_pair, ids, offsets)
