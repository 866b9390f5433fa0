"""Mixers that carry a state of fixed size from token to token instead of keys and values.

``MatrixMemory``            a matrix memory per head with exponential input and forget gates and a running
                            maximum that keeps them in range (the mLSTM cell of xLSTM).
``GatedLinearRecurrence``   a gated branch times a recurrent branch: short causal convolution, block-diagonal
                            gates, a real diagonal recurrence whose decay the gates set (Griffin's recurrent
                            block with its RG-LRU).

Their states are float32 in the state store (``StateNeed``), zero when a sequence starts, and every quantity
that enters a recurrence (gates, decays, their logarithms and exponentials, normalisers) is float arithmetic in
both precisions; only the projections around them run in the activation dtype. A step may bring any number of
rows per sequence: the kernels walk a sequence's rows in order from the state the step before left, so a prompt,
a portion of one and a single token are the same code.
"""

from __future__ import annotations

import torch

from ..cache.spec import StateNeed
from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_part
from .base import Mixer, StepContext, matrix
from .linear import linear


_MAX_SEGMENTS = 8
_CHUNKED_FROM = 8       # steps whose longest sequence brings more rows than this take the chunked matrix-memory kernel


def _vector(n, init="normal"):
    return ((int(n),), VECTOR, init)


class MatrixMemory(Mixer):
    """Per head: ``S <- exp(f + m - m') S + exp(i - m') k v^T``, ``n`` likewise with ``k`` alone, ``m' = max(f + m, i)``,
    read out as ``S^T q / (max(|n . q|, exp(-m')) + 1e-6)`` with ``q`` scaled by ``key_dim^-1/2``; the log gates are
    ``i = cap tanh(. / cap)`` and ``f = logsigmoid(cap tanh(. / cap))`` of two projections with biases. Each head's
    read-out is divided by its root mean square, weighted, gated by ``sigmoid(W_g h)`` and projected back."""

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, gate_cap: float, norm_eps: float):
        self.hidden, self.n_heads, self.key_dim, self.value_dim = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        if not 0 < self.key_dim <= ops.MLSTM_MAX_DIM:
            raise ValueError(f"key_dim must lie in 1..{ops.MLSTM_MAX_DIM}, got {key_dim}")
        if not gate_cap > 0:
            raise ValueError(f"gate_cap must be positive, got {gate_cap}")
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.qk_dim, self.v_dim = self.n_heads * self.key_dim, self.n_heads * self.value_dim
        self.w_in = self.w_gates = self.w_o = self.bias_i = self.bias_f = self.out_norm = None

    def tensor_specs(self):
        return {"q_proj": matrix((self.qk_dim, self.hidden)), "k_proj": matrix((self.qk_dim, self.hidden)),
                "v_proj": matrix((self.v_dim, self.hidden)), "g_proj": matrix((self.v_dim, self.hidden)),
                "o_proj": matrix((self.hidden, self.v_dim)), "out_norm": _vector(self.v_dim, "ones"),
                "i_proj": matrix((self.n_heads, self.hidden)), "i_bias": _vector(self.n_heads),
                "f_proj": matrix((self.n_heads, self.hidden)), "f_bias": _vector(self.n_heads)}

    def load(self, tensors):
        self.w_in = torch.cat([tensors[n] for n in ("q_proj", "k_proj", "v_proj", "g_proj")], dim=0).contiguous()
        self.w_gates = torch.cat([tensors["i_proj"], tensors["f_proj"]], dim=0).contiguous()
        self.w_o = tensors["o_proj"]
        self.bias_i, self.bias_f = tensors["i_bias"].float().contiguous(), tensors["f_bias"].float().contiguous()
        self.out_norm = tensors["out_norm"].float().contiguous()

    def cache_need(self):
        # the normaliser and the maximum once per run of value columns that a workgroup owns, so that no workgroup
        # reads what another has already updated
        runs = -(-self.value_dim // ops.MLSTM_COLUMNS)
        return {"memory": StateNeed((self.n_heads, self.key_dim, self.value_dim)),
                "normaliser": StateNeed((self.n_heads, runs, self.key_dim)), "maximum": StateNeed((self.n_heads, runs))}

    def kernel_modules(self, dtype):
        return ("gemm", "mlstm")

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        rows = h.shape[0]
        proj = linear(h, self.w_in)                                       # q | k | v | g, in the activation dtype
        gates = linear(h, self.w_gates, out_dtype=torch.float32)           # the gates stay float32 from here on
        o_raw = torch.empty((rows, self.n_heads, self.value_dim), dtype=torch.float32, device=h.device)
        # steps of many rows in bfloat16: a chunk of tokens at a time on the matrix cores; single tokens, float32
        # and sizes without 16-byte pieces: token by token in float arithmetic
        chunked = ctx.max_q_len > _CHUNKED_FROM and \
            ops.mlstm_chunks_takes(proj, 0, self.qk_dim, 2 * self.qk_dim, self.key_dim, self.value_dim)
        ops.mlstm_steps(proj, 0, self.qk_dim, 2 * self.qk_dim, gates, self.bias_i, self.bias_f, self.gate_cap,
                        ctx.seq_slot, ctx.cu_rows, ctx.q_len, ctx.n_seqs, line["memory"].state,
                        line["normaliser"].state, line["maximum"].state, o_raw, self.n_heads, self.key_dim,
                        self.value_dim, self.key_dim ** -0.5, writes_cache, chunked=chunked,
                        segments=self._segments(ctx) if chunked else None)
        out = torch.empty((rows, self.v_dim), dtype=h.dtype, device=h.device)
        ops.mlstm_out(o_raw, proj, 2 * self.qk_dim + self.v_dim, self.out_norm, ctx.row_slot, out, self.n_heads,
                      self.value_dim, self.norm_eps)
        return linear(out, self.w_o, allow_partials=True)

    @staticmethod
    def _segments(ctx: StepContext):
        """How the chunked kernel cuts long sequences: into at most ``_MAX_SEGMENTS`` segments of whole chunks each
        (a later segment folds the summaries of all before it, so few are better than many), none for sequences
        of at most two chunks."""
        chunks = -(-ctx.max_q_len // ops.MLSTM_CHUNK)
        if chunks <= 2:
            return None
        seg_rows = ops.MLSTM_CHUNK * max(2, -(-chunks // _MAX_SEGMENTS))
        tile_cu, max_tiles = ctx.tiles(seg_rows)
        return seg_rows, tile_cu, max_tiles

    def flops(self, rows, spans):
        """The projections, and per token and head the update of the memory and its read-out."""
        return super().flops(rows, spans) + 4.0 * rows * self.n_heads * self.key_dim * (self.value_dim + 1)


class GatedLinearRecurrence(Mixer):
    """``y = gelu_tanh(W_y h + b_y)``; ``u = conv(W_x h + b_x)`` over the last ``taps`` tokens per channel; per block of
    channels ``r = sigmoid(A u + a)``, ``i = sigmoid(I u + b)``; ``a = exp(-decay_scale * r * softplus(lam))``;
    ``S <- a S + sqrt(1 - a^2) i u``; output ``W_o (S * y)``."""

    def __init__(self, hidden_size: int, width: int, blocks: int, taps: int, decay_scale: float = 8.0):
        self.hidden, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(taps)
        if self.blocks <= 0 or self.width % self.blocks:
            raise ValueError(f"{width} channels do not split into {blocks} equal blocks")
        if not 1 <= self.taps <= ops.RGLRU_MAX_TAPS:
            raise ValueError(f"the convolution takes 1..{ops.RGLRU_MAX_TAPS} taps, got {taps}")
        self.decay_scale = float(decay_scale)
        self.block_size = self.width // self.blocks
        self.w_in = self.w_o = None

    def tensor_specs(self):
        W, B, bs = self.width, self.blocks, self.block_size
        return {"y_proj": matrix((W, self.hidden)), "y_bias": _vector(W), "x_proj": matrix((W, self.hidden)),
                "x_bias": _vector(W), "conv": matrix((W, self.taps)), "conv_bias": _vector(W),
                "gate_a": matrix((B, bs, bs)), "gate_a_bias": ((B, bs), VECTOR, "normal"),
                "gate_i": matrix((B, bs, bs)), "gate_i_bias": ((B, bs), VECTOR, "normal"), "lam": _vector(W),
                "o_proj": matrix((self.hidden, W))}

    def load(self, tensors):
        self.w_in = torch.cat([tensors["y_proj"], tensors["x_proj"]], dim=0).contiguous()      # y | x
        self.w_o = tensors["o_proj"]
        self.gate_a, self.gate_i = tensors["gate_a"].contiguous(), tensors["gate_i"].contiguous()
        for name in ("y_bias", "x_bias", "conv", "conv_bias", "gate_a_bias", "gate_i_bias", "lam"):
            setattr(self, name, tensors[name].float().contiguous())

    def cache_need(self):
        need = {"state": StateNeed((self.width,))}
        if self.taps > 1:
            need["tail"] = StateNeed((self.taps - 1, self.width))
        return need

    def kernel_modules(self, dtype):
        return ("gemm", "rglru")

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        rows, W = h.shape[0], self.width
        proj = linear(h, self.w_in)
        tail = line["tail"].state if self.taps > 1 else None
        coef = torch.empty((rows, 2, W), dtype=torch.float32, device=h.device)
        ops.rglru_gates(proj, W, self.x_bias, self.conv, self.conv_bias, self.taps, self.gate_a, self.gate_a_bias,
                        self.gate_i, self.gate_i_bias, self.lam, self.decay_scale, ctx.row_slot, ctx.row_seq,
                        ctx.row_pos, ctx.seq_start, tail, coef, W, self.blocks)
        if ctx.max_q_len > ops.RGLRU_TILE:
            # a long prompt: its tiles of tokens side by side (rows of sequences that sit out are not visited)
            out = ctx.kept_zeros((rows, W), h.dtype) if ctx.some_sit_out() else \
                torch.empty((rows, W), dtype=h.dtype, device=h.device)
            tile_cu, max_tiles = ctx.tiles(ops.RGLRU_TILE)
            ops.rglru_scan_tiles(coef, proj, W, 0, self.x_bias, self.y_bias, self.taps, ctx.seq_slot, ctx.cu_rows,
                                 ctx.q_len, tile_cu, max_tiles, ctx.n_seqs, line["state"].state, tail, out, W,
                                 writes_cache)
            return linear(out, self.w_o, allow_partials=True)
        out = torch.empty((rows, W), dtype=h.dtype, device=h.device)
        ops.rglru_scan(coef, proj, W, 0, self.x_bias, self.y_bias, self.taps, ctx.seq_slot, ctx.cu_rows, ctx.q_len,
                       ctx.row_slot, ctx.n_seqs, line["state"].state, tail, out, W, writes_cache)
        return linear(out, self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        return super().flops(rows, spans) + 2.0 * rows * self.width * self.taps


register_part("matrix_memory", MatrixMemory)
register_part("gated_linear_recurrence", GatedLinearRecurrence)
