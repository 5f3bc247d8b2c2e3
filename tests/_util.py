"""Shared builders for the parity tests: seeded K/V, paged pools with shuffled pages, tolerances."""

import torch

# max-abs tolerances of the attention output against the fp32 oracle on identically rounded inputs
ATOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


def rounded(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Round to the device dtype and come back to fp32: what the oracle and the GPU both see."""
    return x.to(dtype).float()


def randn(shape, seed: int, dtype: torch.dtype) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return rounded(torch.randn(shape, generator=g), dtype)


class PagedCase:
    """A sequence of n tokens stored in a paged pool whose pages are scattered (seeded
    permutation) inside a pool with `spare` unused pages.

    k, v        fp32 [n, Hkv, D], already rounded to `dtype`
    page_table  int64 [n_pages]: physical page of logical page i
    pool        torch tensor in `dtype`, NHD [pages, 2, P, Hkv, D] or HND [pages, 2, Hkv, P, D]
    """

    def __init__(self, n, hkv, d, page_size, dtype, layout=0, seed=0, spare=3, shuffle=True,
                 kv=None):
        self.n, self.hkv, self.d, self.page_size, self.dtype, self.layout = n, hkv, d, page_size, dtype, layout
        if kv is None:
            kv = (randn((n, hkv, d), seed * 7 + 1, dtype), randn((n, hkv, d), seed * 7 + 2, dtype))
        self.k, self.v = kv
        self.n_pages = (n + page_size - 1) // page_size
        self.max_pages = self.n_pages + spare
        g = torch.Generator().manual_seed(seed * 7 + 3)
        perm = torch.randperm(self.max_pages, generator=g) if shuffle else torch.arange(self.max_pages)
        self.page_table = perm[: self.n_pages].clone()
        self.last_page_len = (n - 1) % page_size + 1
        pad = self.n_pages * page_size - n
        kp = torch.cat([self.k, torch.zeros(pad, hkv, d)]).view(self.n_pages, page_size, hkv, d)
        vp = torch.cat([self.v, torch.zeros(pad, hkv, d)]).view(self.n_pages, page_size, hkv, d)
        # unused pages and the tail of the last page hold large garbage: reading them shows up
        pool = torch.full((self.max_pages, 2, page_size, hkv, d), 77.0)
        pool[self.page_table, 0] = kp
        pool[self.page_table, 1] = vp
        if pad:
            pool[self.page_table[-1], :, self.last_page_len:] = 77.0
        if layout == 1:
            pool = pool.permute(0, 1, 3, 2, 4).contiguous()
        self.pool = pool.to(dtype)
        self._pool_np = None

    @property
    def pool_np(self):
        """fp32 numpy view of the pool for the oracle (computed once)"""
        if self._pool_np is None:
            self._pool_np = self.pool.float().numpy()
        return self._pool_np

    def slots_of(self, positions: torch.Tensor) -> torch.Tensor:
        """physical slot (page * P + entry) of logical token positions"""
        positions = positions.long()
        return self.page_table[positions // self.page_size] * self.page_size + positions % self.page_size


def rotated(x: torch.Tensor, positions, dtype: torch.dtype, theta: float) -> torch.Tensor:
    """x [N, H, D] fp32 rotated at `positions` by the oracle's float64 closed form, rounded to
    `dtype`: what a fused decode step holds in registers (q) or writes to the cache (k)."""
    import numpy as np

    from oracle import tidal_oracle as orc

    y = orc.rope_closed_form(x.numpy(), np.asarray(positions), theta)
    return rounded(torch.from_numpy(y).float(), dtype)


def within_ulps(got: torch.Tensor, want: torch.Tensor, dtype: torch.dtype, ulps: float = 1.0) -> bool:
    """|got - want| <= ulps units in the last place of `dtype` at want's magnitude"""
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    want = want.float().cpu()
    return bool(((got.float().cpu() - want).abs() <= ulps * ulp * want.abs() + 1e-6).all())


def tolerance_report(got: torch.Tensor, want: torch.Tensor) -> float:
    return (got.float().cpu() - want.float().cpu()).abs().max().item()
