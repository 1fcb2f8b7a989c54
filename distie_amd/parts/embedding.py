"""The two ends of the model: the token embedding, h0[t] = E[ids[t]], and the head,
logits = h W^T without a bias (worker/src/inference/qwen2/model.py:297-303, 375-380). A head that is
tied to the embedding declares no tensor of its own and asks for the embedding's by name, so both use
one buffer (model.py:302-303); a file may still hold a copy under the head's name, which is ignored."""

from __future__ import annotations

from .base import Embedding, Head, ParamSpec, register_part


class TokenEmbedding(Embedding):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.params["vocab_size"])
        self.hidden_size = int(spec.params["hidden_size"])
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, ops, ids, meta):
        return ops.embed(ids, self.weight)


class LinearHead(Head):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.params["vocab_size"])
        self.hidden_size = int(spec.params["hidden_size"])
        self.tied_to = spec.params.get("tied_to")        # full name of the tensor to share, or None
        self.weight = None

    def param_specs(self):
        return {} if self.tied_to else {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def shared_specs(self):
        return {"weight": self.tied_to} if self.tied_to else {}

    def optional_names(self):
        return ["weight"] if self.tied_to else []

    def load(self, tensors) -> None:
        self.weight = tensors["weight"] if self.tied_to else tensors["weight"].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.weight, role="head")

    def forward(self, ops, normed):
        return ops.linear_f32out(normed, self.weight)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LinearHead)
