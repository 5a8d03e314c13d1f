"""Recurrent mixers whose state is a matrix per head."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import Mixer, SlotStateSpec, site_memo
from .registry import register_mixer


@register_mixer("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Linear attention with a decay per key channel.  With ``h`` the layer's input:

        q = W_q h * key_dim^(-1/2),  k = W_k h,  v = W_v h          (heads x key_dim / value_dim)
        alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau)                (heads x key_dim)
        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t   (per head)
        out = W_o (rms_norm_per_head(o) * w_norm * silu(W_g h))

    The state ``S`` (float, ``[heads, key_dim, value_dim]``) lives in the request's slot,
    starts at zero and is carried from step to step.  One packed product gives
    ``[q | k | v | gate | low-rank decay input]`` in float; the decays, the recurrence and the
    per-head norm are 32-bit (``csrc/gla.hip``)."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, heads: int, key_dim: int, value_dim: int, decay_rank: int,
                 tau: float, norm_eps: float):
        if not 0 < key_dim <= 256:
            raise ValueError(f"key_dim {key_dim} must lie in 1..256")
        if tau <= 0:
            raise ValueError("tau must be positive")
        self.width = width
        self.dtype = dtype
        self.heads = heads
        self.key_dim = key_dim
        self.value_dim = value_dim
        self.decay_rank = decay_rank
        self.tau = float(tau)
        self.norm_eps = float(norm_eps)
        self.k_cols = heads * key_dim
        self.v_cols = heads * value_dim
        self._memo_in, self._memo_out = {}, {}

    def _columns(self):
        q_col = 0
        k_col = q_col + self.k_cols
        v_col = k_col + self.k_cols
        gate_col = v_col + self.v_cols
        low_col = gate_col + self.v_cols
        return q_col, k_col, v_col, gate_col, low_col, low_col + self.decay_rank

    def parameters(self):
        total = self._columns()[5]
        return {
            "in.weight": ParamSpec((total, self.width), MATRIX),
            "decay.weight": ParamSpec((self.k_cols, self.decay_rank), MATRIX),
            "decay.bias": ParamSpec((self.k_cols,), VECTOR),
            "norm.gamma": ParamSpec((self.value_dim,), VECTOR),
            "out.weight": ParamSpec((self.width, self.v_cols), MATRIX),
        }

    def bind(self, tensors):
        self.in_weight = tensors["in.weight"]
        self.decay_weight = tensors["decay.weight"]
        self.decay_bias = tensors["decay.bias"]
        self.norm_gamma = tensors["norm.gamma"]
        self.out_weight = tensors["out.weight"]
        self.in_packed = kernels.pack_decode_weight(self.in_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        self._memo_in.clear()
        self._memo_out.clear()

    def cache_spec(self):
        return SlotStateSpec((self.heads, self.key_dim, self.value_dim), torch.float32)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        q_col, k_col, v_col, gate_col, low_col, total = self._columns()
        workspace = ctx.workspace
        proj = workspace.first_rows("gla_proj", total, torch.float32, tokens)
        kernels.linear(x, self.in_weight, None, proj, packed=self.in_packed,
                       memo=site_memo(self._memo_in, workspace), shared=ctx.shared_calls)
        alpha = workspace.first_rows("gla_decay", self.k_cols, torch.float32, tokens)
        kernels.gla_decay(proj, low_col, self.decay_weight, self.decay_bias, self.tau, alpha)
        raw = workspace.first_rows("gla_raw", self.v_cols, torch.float32, tokens)
        kernels.gla_scan(proj, (q_col, k_col, v_col), alpha, cache.state, raw, ctx.cu_tokens,
                         ctx.slots, self.heads, self.key_dim, self.value_dim, self.key_dim ** -0.5,
                         longest=1 if ctx.decode_only else 0)
        gated = workspace.first_rows("gla_out", self.v_cols, self.dtype, tokens)
        kernels.gla_output(raw, self.norm_gamma, self.norm_eps, proj[:, gate_col:gate_col + self.v_cols],
                           gated, self.heads, self.value_dim)
        kernels.linear(gated, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, workspace),
                       shared=ctx.shared_calls)


@register_mixer("lightning_attention")
class LightningAttention(Mixer):
    """Linear attention with one fixed decay per head.  With ``h`` the layer's input:

        q = silu(W_q h),  k = silu(W_k h),  v = silu(W_v h)        (heads x key_dim / value_dim)
        S_t = decay_head * S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t   (per head, no other scale)
        out = W_o (rms_norm(o) * w_norm * sigmoid(W_g h))           (the norm over all heads at once)

    The state ``S`` (float, ``[heads, key_dim, value_dim]``) lives in the request's slot, starts
    at zero and is carried from step to step.  One packed product gives ``[q | k | v | gate]`` in
    float; the activations, the recurrence and the norm are 32-bit (``csrc/gla.hip``, the
    recurrence kernel of gated linear attention with a decay per head)."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, heads: int, key_dim: int, value_dim: int, decays,
                 norm_eps: float):
        if not 0 < key_dim <= 256:
            raise ValueError(f"key_dim {key_dim} must lie in 1..256")
        decays = tuple(float(d) for d in decays)
        if len(decays) != heads:
            raise ValueError(f"{len(decays)} decays for {heads} heads")
        self.width = width
        self.dtype = dtype
        self.heads = heads
        self.key_dim = key_dim
        self.value_dim = value_dim
        self.decays = decays
        self.norm_eps = float(norm_eps)
        self.k_cols = heads * key_dim
        self.v_cols = heads * value_dim
        self._memo_in, self._memo_out = {}, {}
        self._piece_slots = {}

    def parameters(self):
        return {
            "in.weight": ParamSpec((2 * self.k_cols + 2 * self.v_cols, self.width), MATRIX),
            "norm.gamma": ParamSpec((self.v_cols,), VECTOR),
            "out.weight": ParamSpec((self.width, self.v_cols), MATRIX),
        }

    def bind(self, tensors):
        self.in_weight = tensors["in.weight"]
        self.norm_gamma = tensors["norm.gamma"]
        self.out_weight = tensors["out.weight"]
        self.head_decay = torch.tensor(self.decays, dtype=torch.float32, device=self.out_weight.device)
        self.in_packed = kernels.pack_decode_weight(self.in_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        self._memo_in.clear()
        self._memo_out.clear()

    def cache_spec(self):
        return SlotStateSpec((self.heads, self.key_dim, self.value_dim), torch.float32)

    # tokens beyond one per item from which a step's items are cut into pieces of PIECE tokens
    PIECES_FROM = 256
    PIECE = 128

    def _scan_in_pieces(self, proj, columns, raw, ctx, cache, tokens, items):
        """The recurrence of a step with long portions: every piece runs the recurrence kernel
        as an item of its own, first from a zero state (which leaves what the piece adds), then,
        after the pieces of each item have been joined in order, from its true start for the
        outputs.  The walk from token to token is as long as a piece, not as a prompt."""
        workspace = ctx.workspace
        slots = cache.state.shape[0]
        most = workspace.max_rows // self.PIECE + slots          # no step has more pieces
        pieces = tokens // self.PIECE + items
        piece_cu = workspace.flat("lightning_piece_cu", most + 1, torch.int32)
        item_first = workspace.flat("lightning_item_first", slots + 1, torch.int32)
        states = workspace.flat("lightning_piece_states", most * cache.state[0].numel(), torch.float32)
        states = states[:pieces * cache.state[0].numel()].view((pieces,) + tuple(cache.state.shape[1:]))
        own_slots = self._piece_slots.get((workspace.serial, pieces))
        if own_slots is None:
            own_slots = self._piece_slots[(workspace.serial, pieces)] = torch.arange(
                pieces, dtype=torch.int32, device=proj.device)
        kernels.scan_pieces(ctx.cu_tokens, items, self.PIECE, pieces, piece_cu, item_first)
        piece_cu = piece_cu[:pieces + 1]
        states.zero_()
        for turn in range(2):
            kernels.gla_scan(proj, columns, None, states, raw, piece_cu, own_slots, self.heads,
                             self.key_dim, self.value_dim, 1.0, head_decay=self.head_decay)
            if turn == 0:
                kernels.decay_join(states, cache.state, piece_cu, item_first, ctx.slots, self.head_decay)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        k_col, v_col = self.k_cols, 2 * self.k_cols
        gate_col = v_col + self.v_cols
        workspace = ctx.workspace
        proj = workspace.first_rows("lightning_proj", gate_col + self.v_cols, torch.float32, tokens)
        kernels.linear(x, self.in_weight, None, proj, packed=self.in_packed,
                       memo=site_memo(self._memo_in, workspace), shared=ctx.shared_calls)
        raw = workspace.first_rows("lightning_raw", self.v_cols, torch.float32, tokens)
        # single tokens take the activation on their way into the recurrence; for portions, whose
        # recurrence waits for every piece that it stages, a launch ahead of it is faster
        if not ctx.decode_only:
            kernels.silu_columns(proj, 0, gate_col)
        items = ctx.slots.numel()
        if tokens - items >= self.PIECES_FROM:
            self._scan_in_pieces(proj, (0, k_col, v_col), raw, ctx, cache, tokens, items)
        else:
            kernels.gla_scan(proj, (0, k_col, v_col), None, cache.state, raw, ctx.cu_tokens, ctx.slots,
                             self.heads, self.key_dim, self.value_dim, 1.0,
                             longest=1 if ctx.decode_only else 0, head_decay=self.head_decay,
                             silu_inputs=ctx.decode_only)
        gated = workspace.first_rows("lightning_out", self.v_cols, self.dtype, tokens)
        kernels.row_norm_gate(raw, self.norm_gamma, self.norm_eps,
                              proj[:, gate_col:gate_col + self.v_cols], gated)
        kernels.linear(gated, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, workspace),
                       shared=ctx.shared_calls)
