"""A short causal convolution over time on each channel of a projection's output."""

from ..config.plan import StateNeed
from ..ops import kernels
from .base import Part, TensorSpec
from .linear_state import _SequenceArrays


class ShortConvolution(_SequenceArrays, Part):
    """``y_t = sum_j w[:, j] * u_(t - taps + 1 + j)`` per channel, zeros before a request's first
    token, no bias.  The channels of several tensors (``names``: a tensor ``[channels, taps]``
    each) lie side by side in one row.  The last ``taps - 1`` inputs of a request are its state,
    kept in the request's row of a state slot that the mixer which owns this part asks for
    (``state_need``) and zeroed when a request starts, which gives the zeros before its first token.
    Not a mixer: a mixer builds it, runs it between its projection and what follows, and lists it
    among its ``sub_parts`` so that the model hands it its tensors and its step arrays (where each
    request's tokens start).  32-bit throughout; it runs inside ``head_prepare`` as that reads the
    projection's columns (csrc/head_prepare.hip).  No
    counterpart in mlx_lm/models/gpt2.py."""

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, channels, taps, names, prefix=""):
        super().__init__(prefix)
        if taps < 1 or not channels or any(c <= 0 for c in channels) or len(channels) != len(names):
            raise ValueError(f"{taps} taps over channels {channels} of tensors {names}")
        self.channels, self.taps = [int(c) for c in channels], int(taps)
        self.n_channels = sum(self.channels)
        self.names = [self._name(n) for n in names]
        self.state_floats = (self.taps - 1) * self.n_channels
        self.weight = None

    def tensors(self):
        return {n: TensorSpec((c, self.taps), "vector") for n, c in zip(self.names, self.channels)}

    def load(self, tensors):
        import torch

        self.weight = torch.cat([tensors[n] for n in self.names]).contiguous()
        # one tap keeps nothing between steps: the kernel still wants a base address, which it never reads
        self.no_state = self.weight.new_zeros((1, 1)) if not self.state_floats else None

    def state_need(self):
        return StateNeed((self.state_floats,), "float32") if self.state_floats else None

    def ahead(self, ctx, state, offset=0):
        """What ``kernels.head_prepare`` takes as ``conv``: the convolution runs as the heads are read.
        ``state``: the requests' state rows, this part's floats from ``offset`` on."""
        if not self.state_floats:
            state, offset = self.no_state, 0
        single = ctx.array("sequences.longest") == 1
        return kernels.ConvolutionAhead(self.weight, state, offset, ctx.token_req, ctx.array("sequences.starts"), ctx.slot_ids, single)

    def keep_inputs(self, ctx, u, state, offset=0):
        """After the step's rows ``u`` (the convolution's inputs) have been read: the requests' last
        ``taps - 1`` inputs for the next step (nothing to do where every request brought one token:
        the kernel that read them moved them up itself)."""
        if self.taps > 1 and ctx.array("sequences.longest") != 1:
            kernels.conv_state_update(u, 0, self.taps, self.n_channels, state, offset, ctx.array("sequences.starts"),
                                      ctx.array("sequences.lens"), ctx.slot_ids, ctx.n_requests)
