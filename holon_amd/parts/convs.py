"""A short causal filter over time on every channel, with the inputs it still needs kept per request.

y_t[c] = act(sum_j w[c, j] * x_(t - taps + 1 + j)[c] (+ x_t[c])), the last column weighing the current token and
zeros standing before a sequence's first token. A request's last taps - 1 inputs live in its slot
(`SlotState [taps - 1, channels]`, oldest first, in the engine's dtype), so a portion of a prompt or a single decoded
token continues exactly where the step before stopped. HIP form: `csrc/recurrent.hip`."""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from .base import Build, Part, SlotState

_P, _I = ctypes.c_void_p, ctypes.c_int
_DT = {torch.float32: 0, torch.bfloat16: 1}


def causal_conv_plain(x, weight, state, slots, starts, query_start, token_row, n_rows, add_input, silu, in_order=False):
    """x [T, C], weight [C, taps], state [S, taps - 1, C] (updated in place), rows as the step lists them
    (slots/starts [B], query_start [B + 1]). float32 arithmetic, taps added oldest first, one rounding. `in_order`:
    every row has one token and token t is row t (a kernel may then do everything in one launch)."""
    taps = weight.shape[1]
    y = torch.empty_like(x)
    w = weight.float()
    qs, slot_of, start_of = query_start.tolist(), slots.tolist(), starts.tolist()
    for b in range(n_rows):
        lo, hi = qs[b], qs[b + 1]
        old = state[slot_of[b]].float() if start_of[b] > 0 else torch.zeros_like(state[slot_of[b]], dtype=torch.float32)
        seq = torch.cat((old, x[lo:hi].float()), dim=0)              # [taps - 1 + n, C]
        acc = torch.zeros((hi - lo, x.shape[1]), dtype=torch.float32, device=x.device)
        for j in range(taps):
            acc = acc + w[:, j] * seq[j: j + hi - lo]
        if add_input:
            acc = acc + x[lo:hi].float()
        if silu:
            acc = acc * torch.sigmoid(acc)
        y[lo:hi] = acc.to(x.dtype)
        if taps > 1:
            state[slot_of[b]] = seq[seq.shape[0] - (taps - 1):].to(state.dtype)
    return y


def _causal_conv_hip(launch, x, weight, state, slots, starts, query_start, token_row, n_rows, add_input, silu,
                     in_order=False):
    t, c = x.shape
    taps = weight.shape[1]
    if not (x.is_cuda and x.is_contiguous() and x.dtype in _DT and weight.dtype == x.dtype and weight.is_contiguous()
            and weight.shape[0] == c and state.dtype == x.dtype and state.is_contiguous()
            and tuple(state.shape[1:]) == (taps - 1, c) and 1 <= taps <= 16):
        raise ValueError(f"causal_conv: rows {tuple(x.shape)}, taps {tuple(weight.shape)}, state {tuple(state.shape)} "
                         "(contiguous, one dtype, 1 to 16 taps)")
    y = torch.empty_like(x)
    launch(x.data_ptr(), weight.data_ptr(), state.data_ptr(), y.data_ptr(), slots.data_ptr(), starts.data_ptr(),
           query_start.data_ptr(), token_row.data_ptr(), t, n_rows, c, taps, state.shape[0], int(add_input), int(silu),
           _DT[x.dtype], int(bool(in_order) and t == n_rows))
    return y


register_kernel(KernelOp("causal_conv", causal_conv_plain, "holon_causal_conv",
                         [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I], _causal_conv_hip))


class CausalConv(Part):
    """The filter as a part: `weight` [channels, taps]; `add_input` adds the input to the filter's output,
    `silu` applies x * sigmoid(x) last. `name` is the name of its state among its owner's."""

    graph_safe = True

    def __init__(self, build: Build, *, channels: int, taps: int, add_input: bool = False, silu: bool = False,
                 name: str = "conv") -> None:
        super().__init__(build)
        if not 1 <= taps <= 16:
            raise ValueError(f"a causal filter has 1 to 16 taps, got {taps}")
        self.channels, self.taps, self.add_input, self.silu, self.name = channels, int(taps), add_input, silu, name
        self.declare("weight", (channels, taps), init="tap")

    def state(self):
        return [SlotState(self.name, (self.taps - 1, self.channels))]

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        return self.kernels.causal_conv(x, self.weight, site.slot_state[self.name], step.slots, step.starts,
                                        step.query_start, step.token_row, step.n_rows, self.add_input, self.silu,
                                        step.rows.in_order)

    __call__ = forward
