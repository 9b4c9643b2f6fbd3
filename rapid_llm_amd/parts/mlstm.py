"""Matrix-memory recurrence (mLSTM) as a mixer with a fixed-size state per request.

Per head the mixer keeps a matrix ``S [key_dim, value_dim]``, a vector ``n [key_dim]`` and a
running maximum ``m``, all float32, zero when a request begins.  A token brings a query and a
key (``key_dim``), a value (``value_dim``), a log input gate ``i`` and a log forget gate ``f``::

    i = cap * tanh(pre_i / cap)          f = logsigmoid(cap * tanh(pre_f / cap))
    m' = max(f + m, i)
    S' = exp(f + m - m') S + exp(i - m') k v^T         n' likewise with k alone
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)     with q scaled by key_dim^(-1/2)

Each head's ``o`` is divided by its root mean square, the concatenated heads are multiplied
by a weight and by ``sigmoid(gate(x))``, and the output projection follows.

One product makes the packed row ``[q | k | v | gate]`` in the compute type.  The gates'
pre-activations come from a second, small product whose matrix is held in float32 in every
engine and whose result is float32 (a kernel of its own for these few columns; in a bfloat16
engine's steps of few rows the few-row product with float32 results, over the same weights as
bfloat16 where that loses nothing: a product of two bfloat16 numbers is exact in float32), and
everything from there to the finished head outputs is float32 in the kernels
(``csrc/mlstm.hip``).  The state lives in the request's slot (``cache.states``), so portions,
single tokens and batches of both continue where the request's last step stopped.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source, StateSpec
from .linear import Linear


class MatrixMemory(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        key_dim: int,
        value_dim: int,
        gate_cap: float,
        norm_eps: float,
        checkpoint_prefix: str,
        position=None,  # the recurrence knows order by itself
        name: str = "mixer",
        q_name: str = "q",
        k_name: str = "k",
        v_name: str = "v",
        gate_name: str = "g",
        o_name: str = "o",
        norm_name: str = "norm",
        input_gate_name: str = "i",
        forget_gate_name: str = "f",
        input_gate_bias_name: str = "i.b",
        forget_gate_bias_name: str = "f.b",
    ) -> None:
        if not 1 <= key_dim <= ops.MLSTM_MAX_KEY_DIM:
            raise ValueError(f"the recurrence's kernels take key sizes up to {ops.MLSTM_MAX_KEY_DIM}, got {key_dim}")
        if num_heads < 1 or value_dim < 1 or not gate_cap > 0:
            raise ValueError(f"{num_heads} heads of value size {value_dim} with gate cap {gate_cap}")
        self.hidden_size = hidden_size
        self.heads, self.dk, self.dv = num_heads, key_dim, value_dim
        self.cap, self.eps = float(gate_cap), float(norm_eps)
        self.prefix, self.name = checkpoint_prefix, name
        self.names = dict(q=q_name, k=k_name, v=v_name, g=gate_name, o=o_name, norm=norm_name,
                          i=input_gate_name, f=forget_gate_name, ib=input_gate_bias_name,
                          fb=forget_gate_bias_name)
        qk, vv = num_heads * key_dim, num_heads * value_dim
        # columns of q, k, v and the output gate in the packed row, padded to whole groups of 8
        self.columns = (0, qk, 2 * qk, 2 * qk + vv)
        self.pad = -(2 * qk + 2 * vv) % 8
        self.packed = Linear(hidden_size, 2 * qk + 2 * vv + self.pad)
        self.gates = Linear(hidden_size, 2 * num_heads)
        self.o = Linear(vv, hidden_size)
        self.gate_bias = self.norm_weight = None

    def param_specs(self) -> list[ParamSpec]:
        p, n = self.prefix, self.names
        qk, vv, h = self.heads * self.dk, self.heads * self.dv, self.heads
        packed = [Source(p + n["q"], qk), Source(p + n["k"], qk), Source(p + n["v"], vv), Source(p + n["g"], vv)]
        if self.pad:
            packed.append(Source("", self.pad))
        return [
            ParamSpec(self.name + ".packed", (self.packed.out_features, self.hidden_size), "matrix", tuple(packed)),
            ParamSpec(self.name + ".gates", (2 * h, self.hidden_size), "matrix_f32",
                      (Source(p + n["i"], h), Source(p + n["f"], h))),
            ParamSpec(self.name + ".gate_bias", (2 * h,), "vector", (Source(p + n["ib"], h), Source(p + n["fb"], h))),
            ParamSpec(self.name + ".norm", (vv,), "vector", (Source(p + n["norm"], vv),), init="norm"),
            ParamSpec(self.name + ".o", (self.hidden_size, vv), "matrix", (Source(p + n["o"], self.hidden_size),)),
        ]

    def bind(self, params, runtime) -> None:
        self.packed.bind(params[self.name + ".packed"])
        gates = params[self.name + ".gates"]
        self.gates.bind(gates)
        # the same weights as bfloat16 for the few-row product, where they are exactly that
        self.gates_few = None
        if runtime.dtype == torch.bfloat16 and self.hidden_size % 8 == 0:
            narrow = gates.to(torch.bfloat16)
            if torch.equal(narrow.to(torch.float32), gates):
                self.gates_few = Linear(self.hidden_size, 2 * self.heads)
                self.gates_few.bind(narrow)
        self.gate_bias = params[self.name + ".gate_bias"]
        self.norm_weight = params[self.name + ".norm"]
        self.o.bind(params[self.name + ".o"])

    def cache_need(self) -> CacheNeed:
        return CacheNeed(
            "state",
            states=(
                StateSpec("S", (self.heads, self.dk, self.dv), "float32"),
                StateSpec("n", (self.heads, self.dk), "float32"),
                StateSpec("m", (self.heads,), "float32"),
            ),
        )

    @property
    def accepts_scaled_rows(self) -> bool:
        # both products that read the normalised rows must be able to finish the norm
        return self.gates_few is not None and self.packed.takes_scaled_rows()

    def forward(self, x, ctx, cache):
        packed = self.packed(x)
        if self.gates_few is not None and self.gates_few.skinny(x):
            pre = self.gates_few(x, out_dtype=torch.float32)
        else:
            pre = ops.gate_product(x, self.gates.weight)
        out = torch.empty((x.shape[0], self.heads * self.dv), dtype=packed.dtype, device=x.device)
        ops.mlstm(
            packed, self.columns, pre, self.gate_bias, self.norm_weight, out, ctx,
            cache.states["S"], cache.states["n"], cache.states["m"],
            self.heads, self.dk, self.dv, self.cap, self.eps,
        )
        return self.o.deferred(out, ctx)


MIXERS.register("matrix_memory", MatrixMemory)
