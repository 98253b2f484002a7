"""Decode loop captured in a HIP graph.

One decode step of a Mamba stack is a few dozen small kernels per layer (projections at batch
size B, the conv window, the state-update kernel, norms): at decode batch sizes the time goes
into launching them, not into running them.  `GraphedDecoder` records one step of
`LM.step` (or of a bare `Mamba` stack) into a graph once and replays it per token; the
recurrent state and the conv windows live in fixed buffers that the step updates in place, so a
replay allocates nothing and launches everything with one call.

The reference has no counterpart (its `generate` re-runs the whole sequence per token,
mambapy/lm.py:119-155; `MambaBlock.step`, mamba.py:351-382, is the per-token function this
captures).
"""
import torch

from .language_model import LM
from .modules import Mamba


class GraphedDecoder:
    """decoder = GraphedDecoder(model, caches); logits = decoder(token) for every new token.

    model  : LM (input: token ids (B,), output: logits (B, vocab)) or Mamba (input and output
             (B, d_model)).
    caches : list of (h (B, ED, N), window (B, ED, d_conv-1)) per layer, e.g. from
             LM.prefill(...) or Mamba.empty_caches(...); h may be None (zero state).  The
             decoder copies them into its own buffers.
    The returned tensor is the decoder's output buffer: it is overwritten by the next call.
    Weights are read from the model's own tensors at replay time, except the float32 forms of
    the small parameters (A, D, biases, conv and norm weights), which live in per-module buffers
    that an eager forward/step refreshes in place after a weight update; build a new decoder
    (or run one eager step) after changing those.
    """

    def __init__(self, model, caches, warmup: int = 2):
        if isinstance(model, LM):
            self._lm, self._mamba = model, model.mamba
        elif isinstance(model, Mamba):
            self._lm, self._mamba = None, model
        else:
            raise TypeError("GraphedDecoder takes an LM or a Mamba stack")
        p = next(model.parameters())
        cfg = self._mamba.config
        batch = caches[0][1].shape[0]
        self.caches = []
        for h, window in caches:
            hb = torch.zeros(batch, cfg.d_inner, cfg.d_state, dtype=torch.float32, device=p.device)
            if h is not None:
                hb.copy_(h)
            self.caches.append((hb, window.detach().to(p.dtype).clone().contiguous()))
        if self._lm is not None:
            self._inp = torch.zeros(batch, dtype=torch.long, device=p.device)
        else:
            self._inp = torch.zeros(batch, cfg.d_model, dtype=p.dtype, device=p.device)
        self._graph = None
        self._out = None
        # eager warm-up on a side stream (library handles, autotuning), on copies of the state
        saved = [(h.clone(), w.clone()) for h, w in self.caches]
        side = torch.cuda.Stream(device=p.device)
        side.wait_stream(torch.cuda.current_stream(p.device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                self._step()
        torch.cuda.current_stream(p.device).wait_stream(side)
        for (h, w), (h0, w0) in zip(self.caches, saved):
            h.copy_(h0)
            w.copy_(w0)
        torch.cuda.synchronize(p.device)
        self._graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self._graph):
            self._out = self._step()
        # the capture itself does not execute: state is still the caller's
        torch.cuda.synchronize(p.device)

    def _step(self):
        if self._lm is not None:
            x = self._mamba.step_(self._lm.embedding(self._inp), self.caches)
            return self._lm.lm_head(self._lm.norm_f(x))
        return self._mamba.step_(self._inp, self.caches)

    @torch.no_grad()
    def __call__(self, inp):
        self._inp.copy_(inp)
        self._graph.replay()
        return self._out
