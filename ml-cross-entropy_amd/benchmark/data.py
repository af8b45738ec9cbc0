"""Synthetic inputs (ref: benchmark/data/data.py, benchmark/data/randn.py:7-38, benchmark/data/__init__.py:9-40).

The reference's named data sets run a downloaded language model over a downloaded corpus to get
embeddings; here a name only selects the *shape* of that model's head (tokens, hidden size,
vocabulary, soft-cap), filled with E ~ N(0, 1), C ~ N(0, 0.02), uniform labels from a fixed seed.
"""

from dataclasses import dataclass
from typing import Callable, Dict, Optional

import torch


@dataclass
class Data:
    embedding: torch.Tensor
    classifier: torch.Tensor
    targets: torch.Tensor
    softcap: Optional[float] = None


def randn_generate(device="cuda", dtype=torch.bfloat16, M=256, N=512, D=128) -> Data:
    """The reference's random generator: both matrices ~ N(0, 1) / D^(1/4), the first rows of the
    classifier copied from the embeddings so that some logits are large (ref: benchmark/data/randn.py:31-38)."""
    w = torch.randn(N, D, device=device, dtype=dtype) / D**0.25
    x = torch.randn(M, D, device=device, dtype=dtype) / D**0.25
    w[:M] = x[: min(N, M)]
    targets = torch.randint(0, N, size=(M,), device=device)
    targets = targets[torch.randperm(M, device=targets.device)]
    return Data(x, w, targets)


def _head_shaped(tokens: int, hidden: int, vocab: int, softcap: Optional[float]) -> Callable[..., Data]:
    def generate(device="cuda", dtype=torch.bfloat16) -> Data:
        g = torch.Generator(device="cpu").manual_seed(0)
        e = torch.randn((tokens, hidden), generator=g).to(device=device, dtype=dtype)
        c = torch.empty((vocab, hidden), device=device, dtype=dtype)
        for s in range(0, vocab, 32000):  # bounded host memory
            n = min(32000, vocab - s)
            c[s : s + n] = (torch.randn((n, hidden), generator=g) * 0.02).to(device=device, dtype=dtype)
        t = torch.randint(0, vocab, (tokens,), generator=g).to(device)
        return Data(e, c, t, softcap)

    return generate


generators: Dict[str, Callable[..., Data]] = {
    "randn": randn_generate,
    # shapes of the heads the reference's data sets come from, 8192 tokens each
    "gemma2": _head_shaped(8192, 2304, 256000, 30.0),
    "llama3": _head_shaped(8192, 4096, 128256, None),
    "mistral-nemo": _head_shaped(8192, 5120, 131072, None),
    "phi3.5": _head_shaped(8192, 3072, 32064, None),
}


def generator(name: str) -> Callable[..., Data]:
    if name not in generators:
        raise ValueError(f"Unknown test data {name!r}; known: {sorted(generators)}")
    return generators[name]
