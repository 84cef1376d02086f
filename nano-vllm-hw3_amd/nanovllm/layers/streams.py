"""Multi-stream residual ("hyper-connections"): S copies of the residual stream instead of one.  A sublayer reads a
learned weighted sum of the streams and its output is written back to every stream with a learned weight while the
streams are mixed by a learned S x S matrix.  With S = 1 and all weights 1 this is the ordinary residual sum."""
import torch
from torch import nn


class StreamPort(nn.Module):
    """The weights of one sublayer's access to the streams: ``w_in`` [S] (read), ``mix`` [S, S] ([from, to]) and
    ``out`` [S] (write).  Always float32: the streams are."""

    def __init__(self, streams: int, learned: bool = True):
        super().__init__()
        self.streams = streams
        self.learned = learned
        f32 = dict(dtype=torch.float32)
        self.w_in = nn.Parameter(torch.ones(streams, **f32), requires_grad=False)
        self.mix = nn.Parameter(torch.eye(streams, **f32), requires_grad=False)
        self.out = nn.Parameter(torch.ones(streams, **f32), requires_grad=False)
