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
    def prefill(self, tokens):
        """Run the prompt once; returns (logits of the last position (B, vocab), caches)."""
        x, caches = self.mamba(self.embedding(tokens), return_caches=True)
        return self.lm_head(self.norm_f(x[:, -1])), caches

    @torch.no_grad()
    def step(self, token, caches):
        """token : (B,) int64 -> (logits (B, vocab), caches); one decode step per call."""
        x, caches = self.mamba.step(self.embedding(token), caches)
        return self.lm_head(self.norm_f(x)), caches

    @torch.no_grad()
    def generate(self, prompt, num_tokens: int, sample: bool = False, temperature: float = 1.0):
        """Greedy (or sampled) continuation of `prompt` (B, L): one prefill, then O(1) steps."""
        logits, caches = self.prefill(prompt)
        out = [prompt]
        for _ in range(num_tokens):
            if sample:
                probs = torch.softmax(logits.float() / temperature, dim=-1)
                nxt = torch.multinomial(probs, 1).squeeze(1)
            else:
                nxt = logits.argmax(-1)
            out.append(nxt.unsqueeze(1))
            logits, caches = self.step(nxt, caches)
        return torch.cat(out, dim=1)
