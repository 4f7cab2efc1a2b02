"""Seeded synthetic inputs of the analog SigmaMoE layer, shared by the benchmark and the tests.

Distributions follow the reference's own test set-up (test_moe_layer_aihwkit_lightning.py:82-90, 232: standard-normal
tokens, a sigmoid gate over a linear router, top-k without sorting); weights are scaled by 1/sqrt(fan-in)."""
import torch


def make_problem(seed, T, D, E, F, k, dtype=torch.float32, routing="router", device="cpu"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, D, generator=g)
    keys = torch.randn(E, D, F, generator=g) / D ** 0.5
    values = torch.randn(E, F, D, generator=g) / F ** 0.5
    if routing == "router":
        router = torch.randn(E, D, generator=g) / D ** 0.5
        gate, idx = torch.sigmoid(x @ router.t()).topk(k, dim=-1, sorted=False)
    elif routing == "uniform":      # every expert gets exactly T*k/E rows (T*k a multiple of E), in shuffled order
        # flat position r of the k-head list goes to expert r % E: a token's k experts are consecutive, hence
        # distinct for k <= E; the tokens are then shuffled, which keeps every expert's count
        base = (torch.arange(T * k) % E).reshape(T, k)
        idx = base[torch.randperm(T, generator=g)]
        gate = torch.rand(T, k, generator=g) * 0.5 + 0.25
    elif routing == "near_uniform":  # k consecutive experts from a random start per token: counts T*k/E +- a few percent
        base = (torch.arange(T * k) % E).reshape(T, k)
        shift = torch.randint(0, E, (T, 1), generator=g)
        idx = (base + shift) % E
        gate = torch.rand(T, k, generator=g) * 0.5 + 0.25
    elif routing == "zipf":         # logits biased so that load follows Zipf(1.2)
        p = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        logits = torch.randn(T, E, generator=g) + torch.log(p / p.sum())
        gate, idx = torch.sigmoid(logits).topk(k, dim=-1, sorted=False)
    else:
        raise ValueError(routing)
    dy = torch.randn(T, D, generator=g)
    cast = lambda t: t.to(dtype).to(device)
    return dict(x=cast(x), keys=cast(keys), values=cast(values), idx=idx.to(device), gate=cast(gate), dy=cast(dy))
