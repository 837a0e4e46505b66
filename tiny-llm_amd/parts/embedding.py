"""Token embedding (a row gather, no scale: tiny_llm/ops/cuda/embedding.cu:10-29)
and the output head (logits = xn W^T at the wanted rows only:
tiny_llm/ops/cuda/gemm_q1_helper.cu:99-124).  A tied head uses the embedding
table; the reference never reads `tie_word_embeddings`."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Embedding, Head, StateSpec, WeightSpec, register_embedding, register_head
from .norm import LazyNorm


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, vocab_size: int, hidden_size: int, weight_name: str = "weight",
                 scale: float = 1.0):
        """scale: a constant the rows are multiplied by (in float32)."""
        super().__init__(prefix, dtype, device)
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.tensor_name = f"{prefix}.{weight_name}" if weight_name else prefix
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(self.tensor_name, (self.vocab_size, self.hidden_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor_name].contiguous()

    def forward(self, tokens: torch.Tensor, ctx=None) -> torch.Tensor:
        out = ops.scratch("residual", (tokens.numel(), self.hidden_size), torch.float32, tokens.device)
        return ops.embedding(tokens, self.weight, out, self.scale)


class PairEmbedding(Embedding):
    """x = table[token] * scale + pairs[(previous token * mul_prev + token * mul_cur) mod buckets]: a second
    table of `buckets` + 1 rows looked up by a hash of the token and the one before it in its request; a
    request's first token has none before it and takes the last row.  The previous token is per-request
    state: one int32 per state slot, read for the first token a request brings in a step and overwritten
    with the last one it brings (the decoder hands the state tensor to `forward`)."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int,
                 mul_cur: int, scale: float = 1.0, weight_name: str = "weight", pairs_name: str = "pairs"):
        """pairs_name: the pair table's tensor name (whole, not below the prefix)."""
        super().__init__(prefix, dtype, device)
        self.vocab_size, self.hidden_size, self.buckets = int(vocab_size), int(hidden_size), int(buckets)
        self.mul_prev, self.mul_cur, self.scale = int(mul_prev), int(mul_cur), float(scale)
        if self.buckets <= 0:
            raise ValueError(f"{prefix}: the pair table needs at least one bucket")
        self.tensor_name = f"{prefix}.{weight_name}" if weight_name else prefix
        self.pairs_name = pairs_name
        self.weight: Optional[torch.Tensor] = None
        self.pairs: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(self.tensor_name, (self.vocab_size, self.hidden_size)),
                WeightSpec(self.pairs_name, (self.buckets + 1, self.hidden_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor_name].contiguous()
        self.pairs = tensors[self.pairs_name].contiguous()

    def state_spec(self) -> StateSpec:
        return StateSpec((1,), torch.int32)

    def forward(self, tokens: torch.Tensor, ctx=None, state: Optional[torch.Tensor] = None) -> torch.Tensor:
        if ctx is None or state is None:
            raise ValueError(f"{self.prefix}: the pair table needs the step's context and the requests' state")
        out = ops.scratch("residual", (tokens.numel(), self.hidden_size), torch.float32, tokens.device)
        return ops.embedding_pairs(tokens, ctx.positions, ctx.req_of_token, ctx.cu_seqlens_q, ctx.state_slots, state,
                                   self.weight, self.pairs, out, self.mul_prev, self.mul_cur, self.scale)


class LMHead(Head):
    graph_safe = True
    accepts_lazy_norm = True

    def __init__(self, prefix, dtype, device, *, vocab_size: int, hidden_size: int, tied_to: str = None,
                 weight_name: str = "weight", softcap: float = 0.0, tied_exact: bool = False):
        """softcap c > 0: logits <- c * tanh(logits / c)."""
        super().__init__(prefix, dtype, device)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to          # weight prefix of the embedding whose table this head shares
        self.tied_exact = bool(tied_exact)
        self.tensor_name = f"{prefix}.{weight_name}" if weight_name else prefix
        self.softcap = float(softcap or 0.0)
        if self.softcap < 0:
            raise ValueError("the soft cap of the logits must be positive (0: none)")
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        # `tied_to` names the embedding's weight prefix (its table is `<prefix>.weight`), or, with a name that the
        # checkpoint holds as it stands (an embedding whose prefix IS the tensor), that tensor
        alias = None
        if self.tied_to:
            alias = self.tied_to if self.tied_exact else f"{self.tied_to}.weight"
        return [WeightSpec(self.tensor_name, (self.vocab_size, self.hidden_size), alias_of=alias)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor_name].contiguous()

    def forward(self, h) -> torch.Tensor:
        """h: activations [n, H], or a LazyNorm whose norm rides in the product."""
        if isinstance(h, LazyNorm):
            out = torch.empty((h.num_rows, self.vocab_size), dtype=torch.float32, device=h.x.device)
            out = h.linear(self.weight, out)
        else:
            out = torch.empty((h.shape[0], self.vocab_size), dtype=torch.float32, device=h.device)
            out = ops.linear(h, self.weight, out)
        return ops.softcap(out, self.softcap) if self.softcap else out


register_embedding("token_embedding", TokenEmbedding)
register_embedding("pair_embedding", PairEmbedding)
register_head("lm_head", LMHead)
