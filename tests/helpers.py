"""Seeded input builders shared by the parity tests (CPU generator, then moved,
so the oracle and the HIP path see identical bits)."""

from __future__ import annotations

import torch


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def rel_l2(actual: torch.Tensor, expected: torch.Tensor) -> float:
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    return ((a - e).norm() / e.norm().clamp_min(1e-30)).item()


def routing(seed: int, num_tokens: int, slots: int, num_banks: int, zero_frac: float = 0.15):
    """Random ids ``[T, slots]`` and fp32 weights with some exact zeros, as the
    reference's own kernel tests draw them (tests/test_triton_expert_dispatch.py:119-139)."""

    g = gen(seed)
    ids = torch.randint(0, num_banks, (num_tokens, slots), generator=g)
    weights = torch.rand(num_tokens, slots, generator=g)
    weights[torch.rand(num_tokens, slots, generator=g) < zero_frac] = 0.0
    return ids, weights


def bank_weights(seed: int, num_banks: int, d: int, h: int, std: float, dtype=torch.float32):
    g = gen(seed)
    w_up = (torch.randn(num_banks, d, h, generator=g) * std).to(dtype)
    w_gate = (torch.randn(num_banks, d, h, generator=g) * std).to(dtype)
    w_down = (torch.randn(num_banks, h, d, generator=g) * std).to(dtype)
    return w_up, w_gate, w_down


def zipf_ids(seed: int, num_tokens: int, slots: int, num_banks: int, alpha: float = 1.2):
    """Skewed routing: bank popularity ~ rank^-alpha over a seeded permutation,
    heavy enough that several banks get no row."""

    g = gen(seed)
    rank = torch.randperm(num_banks, generator=g).double() + 1.0
    p = rank.pow(-alpha * 2.5)
    p = p / p.sum()
    return torch.multinomial(p, num_tokens * slots, replacement=True, generator=g).view(
        num_tokens, slots
    )


def tile_tables(tile_table: torch.Tensor, rows_pad: int, num_banks: int):
    """The three tables of a tile_table buffer as ``(bank, row0, nrows)`` triples of their
    live entries: 128-row tiles, balanced tiles of up to 160 rows, balanced tiles of up to
    320 rows.
    Also returns a copy of the buffer with every unspecified entry (beyond each table's
    count) zeroed, for bit-for-bit comparisons of two builds."""

    tt = tile_table.detach().cpu().clone()
    caps = (rows_pad // 128 + num_banks + 2, rows_pad // 128 + num_banks + 2,
            rows_pad // 256 + num_banks + 2)
    assert tt.numel() == sum(3 * c + 1 for c in caps)
    out, base = [], 0
    for cap in caps:
        n = int(tt[base + 3 * cap])
        assert 0 <= n <= cap
        out.append((tt[base:base + n].clone(), tt[base + cap:base + cap + n].clone(),
                    tt[base + 2 * cap:base + 2 * cap + n].clone()))
        for part in range(3):
            tt[base + part * cap + n:base + (part + 1) * cap] = 0
        base += 3 * cap + 1
    return out, tt
