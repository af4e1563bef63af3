"""Seeded synthetic workloads: the five benchmark configurations, at full size or shrunk.

Shapes: (1) 8 experts x 128 rows, 128 -> 128, the CPU-sized plumbing case;
(2) Mixtral-8x7B expert FFN w1: 8 experts, 16384 tokens routed top-2 -> 32768 rows,
4096 -> 14336; (3) fine-grained ragged MoE: 64 experts, 49152 rows, 2048 -> 1408,
Zipf(1.2) sizes with at least four empty experts; (4) the weight-gradient layout alone:
8 experts x 4096 rows, c (8, 4096, 14336); (5) DeepSeek-V3-style share: 256 experts,
65536 rows, 7168 -> 2048 with b stored transposed (256, 2048, 7168).

`shrink` divides the row count and both hidden sizes (kept multiples of 8) so the same
generators serve the small parity cases.
"""
from dataclasses import dataclass

import torch


@dataclass
class Workload:
    name: str
    a: torch.Tensor            # (tokens, hidden_in)
    b: torch.Tensor            # (E, hidden_in, hidden_out) or (E, hidden_out, hidden_in) if trans_b
    grad: torch.Tensor         # (tokens, hidden_out), the upstream gradient of the forward output
    batch_sizes: torch.Tensor  # int64 (E,), on the CPU
    trans_b: bool
    gemms: tuple               # which of "fwd", "agrad", "bgrad" the configuration times

    @property
    def tokens(self):
        return self.a.shape[0]

    @property
    def hidden_in(self):
        return self.a.shape[1]

    @property
    def hidden_out(self):
        return self.grad.shape[1]

    def flops_per_gemm(self):
        return 2 * int(self.batch_sizes.sum()) * self.hidden_in * self.hidden_out

    def bytes_per_gemm(self):
        """Each operand read once and the output written once, 2 bytes per element."""
        t = int(self.batch_sizes.sum())
        e = self.batch_sizes.numel()
        return 2 * (t * self.hidden_in + e * self.hidden_in * self.hidden_out + t * self.hidden_out)


def _round8(x):
    return max(8, (int(x) // 8) * 8)


def _randn(shape, gen, device, scale):
    # generated on `device` in fp32 chunks to bound the transient memory
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(-1)
    step = 1 << 26
    for s in range(0, flat.numel(), step):
        n = min(step, flat.numel() - s)
        flat[s:s + n] = (torch.randn(n, generator=gen, device=device) * scale).to(torch.bfloat16)
    return out


def router_sizes(tokens, experts, top_k, gen):
    """Multinomial top-k routing over the softmax of random logits (mild skew)."""
    logits = torch.randn(tokens, experts, generator=gen)
    idx = torch.multinomial(torch.softmax(logits, -1), top_k, replacement=False, generator=gen)
    return torch.bincount(idx.flatten(), minlength=experts).to(torch.int64)


def zipf_sizes(rows, experts, s, empty, gen):
    """Zipf(s) weights over a random permutation of the experts, `empty` of them forced to
    zero, rounded to integers that sum to `rows` (largest remainder)."""
    perm = torch.randperm(experts, generator=gen)
    w = 1.0 / torch.arange(1, experts + 1, dtype=torch.float64) ** s
    w[experts - empty:] = 0.0
    weights = torch.zeros(experts, dtype=torch.float64)
    weights[perm] = w
    exact = weights / weights.sum() * rows
    sizes = exact.floor().to(torch.int64)
    rem = rows - int(sizes.sum())
    order = torch.argsort(exact - sizes.to(torch.float64), descending=True)
    sizes[order[:rem]] += 1
    assert int(sizes.sum()) == rows and int((sizes == 0).sum()) >= empty
    return sizes


def poisson_sizes(rows, experts, gen):
    """Poisson(rows / experts) per expert, then +-1 on random experts until the sum is `rows`."""
    sizes = torch.poisson(torch.full((experts,), rows / experts), generator=gen).to(torch.int64)
    diff = rows - int(sizes.sum())
    while diff != 0:
        e = int(torch.randint(experts, (1,), generator=gen))
        if diff > 0:
            sizes[e] += 1
            diff -= 1
        elif sizes[e] > 0:
            sizes[e] -= 1
            diff += 1
    return sizes


def make(config, device="cuda", shrink=1, seed=0):
    cpu_gen = torch.Generator().manual_seed(seed)
    dev_gen = torch.Generator(device=device).manual_seed(seed)
    if config == 1:
        e, rows, hin, hout, trans_b, scale = 8, 1024, 128, 128, False, 1.0
        sizes = torch.full((e,), 128, dtype=torch.int64)
        gemms = ("fwd", "agrad", "bgrad")
    elif config == 2:
        e, hin, hout, trans_b, scale = 8, _round8(4096 // shrink), _round8(14336 // shrink), False, 0.02
        sizes = router_sizes(16384 // shrink, e, 2, cpu_gen)
        rows = int(sizes.sum())
        gemms = ("fwd", "agrad", "bgrad")
    elif config == 3:
        e, rows, hin, hout, trans_b, scale = 64, 49152 // shrink, _round8(2048 // shrink), _round8(1408 // shrink), False, 0.02
        sizes = zipf_sizes(rows, e, 1.2, 4, cpu_gen)
        gemms = ("fwd",)
    elif config == 4:
        e, hin, hout, trans_b, scale = 8, _round8(4096 // shrink), _round8(14336 // shrink), False, 0.02
        sizes = torch.full((e,), 4096 // shrink, dtype=torch.int64)
        rows = int(sizes.sum())
        gemms = ("bgrad",)
    elif config == 5:
        e, rows, hin, hout, trans_b, scale = 256, 65536 // shrink, _round8(7168 // shrink), _round8(2048 // shrink), True, 0.02
        sizes = poisson_sizes(rows, e, cpu_gen)
        gemms = ("fwd", "agrad", "bgrad")
    else:
        raise ValueError("config must be 1..5")
    a = _randn((rows, hin), dev_gen, device, scale)
    b = _randn((e, hout, hin) if trans_b else (e, hin, hout), dev_gen, device, scale)
    grad = _randn((rows, hout), dev_gen, device, scale)
    return Workload(f"config{config}" + (f"/shrink{shrink}" if shrink != 1 else ""), a, b, grad,
                    sizes, trans_b, gemms)
