"""Language-model wrapper around the Mamba backbone (the reference's `LM`, which its README
calls MambaLM): embedding -> Mamba -> final RMSNorm -> untied linear head
(mambapy/lm.py:20-41, 97-117, 273-279).  state_dict keys: embedding.weight, mamba.layers.*,
norm_f.weight, lm_head.weight.

Only what the scan path needs is restated: forward, the non-muP initialisation and a
prefill/step pair that hands the scan's final state to the decode kernel (the reference's
`generate` re-runs the whole sequence for every new token, lm.py:119-155).  The Hugging Face
loader, the optimizer groups and muP initialisation are out of scope.
"""
import math

import torch
import torch.nn as nn

from .modules import Mamba, MambaConfig, RMSNorm


class LM(nn.Module):
    def __init__(self, model_config: MambaConfig, vocab_size: int, pad_vocab_size_multiple: int = None):
        super().__init__()
        if pad_vocab_size_multiple is not None and vocab_size % pad_vocab_size_multiple != 0:
            vocab_size += pad_vocab_size_multiple - vocab_size % pad_vocab_size_multiple
        if not isinstance(model_config, MambaConfig):
            raise NotImplementedError("only MambaConfig backbones are supported")
        if model_config.mup:
            raise NotImplementedError("muP initialisation is not part of this package")
        self.config = model_config
        self.vocab_size = vocab_size
        self.embedding = nn.Embedding(vocab_size, model_config.d_model, padding_idx=0)
        self.mamba = Mamba(model_config)
        self.norm_f = RMSNorm(model_config.d_model, model_config.rms_norm_eps, model_config.mup)
        self.lm_head = nn.Linear(model_config.d_model, vocab_size, bias=False)

        # N(0, base_std) for every Linear / Embedding weight, zero biases (this also resets
        # dt_proj, as in the reference), then the residual-path scaling of out_proj
        std = model_config.base_std
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, mean=0.0, std=std)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
            elif isinstance(m, nn.Embedding):
                nn.init.normal_(m.weight, mean=0.0, std=std)
        for name, p in self.named_parameters():
            if name.endswith("mixer.out_proj.weight"):
                nn.init.normal_(p, mean=0.0, std=std / math.sqrt(2 * model_config.n_layers))

    def forward(self, tokens):
        """tokens : (B, L) int64 -> logits (B, L, vocab)."""
        x = self.mamba(self.embedding(tokens))
        return self.lm_head(self.norm_f(x))

    @torch.no_grad()
    def prefill(self, tokens, caches=None):
        """Run the prompt once; returns (logits of the last position (B, vocab), caches).  With
        `caches` (from an earlier prefill or step) the prompt continues that sequence, so a long
        prompt can be fed in pieces."""
        x, caches = self.mamba(self.embedding(tokens), caches=caches, return_caches=True)
        return self.lm_head(self.norm_f(x[:, -1])), caches

    @torch.no_grad()
    def step(self, token, caches):
        """token : (B,) int64 -> (logits (B, vocab), caches); one decode step per call."""
        x, caches = self.mamba.step(self.embedding(token), caches)
        return self.lm_head(self.norm_f(x)), caches

    def generate(self, prompt, num_tokens: int, sample: bool = True, top_k: int = None, temperature: float = 1.0):
        """The reference's call (mambapy/lm.py:119-155), same arguments, defaults and result:
        prompt (B, L) -> the num_tokens generated tokens (B, num_tokens) on the prompt's device;
        sampling (optionally restricted to the top_k most likely tokens) unless sample=False; the
        module is put in eval mode for the call and back in train mode afterwards, as there.
        Where the reference runs the whole sequence through forward again for every token, this
        runs the prompt once and then one state-update step per token."""
        if num_tokens <= 0:
            # nothing is appended and the reference's final slice `generated[:, -num_tokens:]` then
            # returns the prompt (from position -num_tokens on); the module ends in train mode there too
            self.train()
            return prompt.clone()[:, -num_tokens:]
        if top_k is not None:
            top_k = min(top_k, self.vocab_size)
        input_device = prompt.device
        prompt = prompt.to(self.embedding.weight.device)
        self.eval()
        out = []
        with torch.no_grad():
            logits, caches = self.prefill(prompt)
            for i in range(num_tokens):
                if sample:
                    probs = torch.softmax(logits.float() / temperature, dim=-1)
                    if top_k is not None:
                        values, _ = torch.topk(probs, k=top_k)
                        probs[probs < values[:, -1, None]] = 0
                        probs = probs / probs.sum(dim=1, keepdim=True)
                    nxt = torch.multinomial(probs, num_samples=1).squeeze(1)
                else:
                    nxt = logits.argmax(dim=-1)
                out.append(nxt.unsqueeze(1))
                if i + 1 < num_tokens:          # the state after the last token is not needed
                    logits, caches = self.step(nxt, caches)
        self.train()
        return torch.cat(out, dim=1).to(input_device)
