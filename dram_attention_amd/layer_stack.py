"""A stack of independent DRAM Attention layers stepped together.

The reference's model walks its layers one after the other on one stream
(evaluation/dram-attention/model.py:265-274, 305-317); each layer's decode step
is page scoring, ordered top-k and the LRU update (no host-link traffic), then
the page stream and attention (bound by the host link).  In an attention-only
stack the layers' queries do not depend on each other, so the first half of
layer i+1 can run while layer i's pages are still crossing the host link: the
link then never waits for a selection.

``AttentionStack.generate`` issues the first halves (and the final merge of each
layer's attention partials) on a side stream and the page stream + attention
launches on the caller's stream, tied together by events;
every layer runs exactly the launches it runs alone, on its own buffers, so the
results have the same bits as stepping the layers one by one.  All streams have
the default priority.  The step has no host synchronisation and can be
captured into one HIP graph per model step (the side stream forks from and
joins the capturing stream).
"""

from __future__ import annotations

from typing import List, Sequence

import torch

from .dram_attention import DRAMAttention


class AttentionStack(torch.nn.Module):
    """``layers``: DRAMAttention modules whose caches are initialised (each with its
    own page cache); ``pipelined``: overlap layer i's page stream with the
    selection of the layers after it."""

    def __init__(self, layers: Sequence[DRAMAttention], pipelined: bool = True):
        super().__init__()
        self.layers = torch.nn.ModuleList(layers)
        self.pipelined = pipelined
        self._side = None
        self._events: List[torch.cuda.Event] = []
        self._stream_done: List[torch.cuda.Event] = []

    def generate(self, xqs: Sequence[torch.Tensor], xks: Sequence[torch.Tensor],
                 xvs: Sequence[torch.Tensor], start_pos) -> List[torch.Tensor]:
        """One decode step of every layer.  xqs[i] (1,1,Hq,D), xks[i]/xvs[i] (1,1,Hkv,D)
        are layer i's inputs; ``start_pos`` (int or int32 device tensor) is shared.
        Returns the layers' outputs, each (1,1,Hq,D)."""
        n = len(self.layers)
        if not (len(xqs) == len(xks) == len(xvs) == n):
            raise ValueError(f"{n} layers need {n} query/key/value tensors each")
        if not self.pipelined or n < 2 or not xqs[0].is_cuda:
            return [layer(xq, xk, xv, start_pos=start_pos, stage="generate")
                    for layer, xq, xk, xv in zip(self.layers, xqs, xks, xvs)]
        dev = xqs[0].device
        main = torch.cuda.current_stream(dev)
        if self._side is None:
            self._side = torch.cuda.Stream(device=dev)      # default priority
        while len(self._events) < n:
            self._events.append(torch.cuda.Event())
        while len(self._stream_done) < n:
            self._stream_done.append(torch.cuda.Event())
        side = self._side
        selected_ev, streamed_ev = self._events, self._stream_done
        side.wait_stream(main)          # inputs are ready; the previous step has finished
        selected = [None] * n
        with torch.cuda.stream(side):
            selected[0] = self.layers[0].select_(xqs[0])
            selected_ev[0].record(side)
        outs = []
        for i, layer in enumerate(self.layers):
            if i + 1 < n:               # the selection runs one layer ahead of the page streams
                with torch.cuda.stream(side):
                    selected[i + 1] = self.layers[i + 1].select_(xqs[i + 1])
                    selected_ev[i + 1].record(side)
            main.wait_event(selected_ev[i])     # this layer's miss list is complete
            out, merge = layer.attend_(xqs[i], xks[i], xvs[i], start_pos, selected[i],
                                       defer_merge=True)
            outs.append(out)
            if merge is not None:
                # the final merge leaves the stream that owns the host link: the next
                # layer's pages start moving as soon as this layer's have landed
                streamed_ev[i].record(main)
                with torch.cuda.stream(side):
                    side.wait_event(streamed_ev[i])
                    merge()
        main.wait_stream(side)          # join: every merge has written its output
        return outs
