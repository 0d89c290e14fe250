"""Seeded synthetic inputs for the five benchmark shapes of the paged-attention path.

All values are drawn on the CPU from ``torch.Generator().manual_seed(0x5EED0000 + config)``:
fp32 N(0,1) rounded to bf16 for q / k / v and for every pool row (unreferenced rows hold
noise too, so stray reads show up), request lengths with ``torch.randint``, and the page
table as one ``torch.randperm`` of the pool's pages consumed request by request.  Token ``t``
of a request lives in slot ``page_table[t // page_size] * page_size + t % page_size``;
``kv_indices`` is that expansion at token granularity, which is what the operators take.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, replace
from typing import List, Optional

import torch

from . import roofline

SEED_BASE = 0x5EED0000
MAX_KV_SPLITS = 32


@dataclass
class PagedWorkload:
    name: str
    kind: str  # "decode" | "prefill"
    n_q: int
    n_kv: int
    head_dim: int
    page_size: int
    sm_scale: float
    kv_lens: List[int]
    extend_lens: List[int]  # all ones for decode
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    kv_indptr: torch.Tensor
    kv_indices: torch.Tensor
    # decode only
    num_kv_splits: Optional[torch.Tensor] = None
    max_kv_splits: int = MAX_KV_SPLITS
    # prefill only
    qo_indptr: Optional[torch.Tensor] = None
    prefix_lens: Optional[torch.Tensor] = None
    max_len_extend: int = 1
    is_cross_attention: bool = False
    sliding_window_size: int = 0
    # rows to store before attending (prefill with store); None when the pool is pre-filled
    new_k: Optional[torch.Tensor] = None
    new_v: Optional[torch.Tensor] = None
    out_loc: Optional[torch.Tensor] = None

    @property
    def batch(self) -> int:
        return len(self.kv_lens)

    @property
    def prefixes(self) -> List[int]:
        return [l - e for l, e in zip(self.kv_lens, self.extend_lens)]

    def to(self, device) -> "PagedWorkload":
        moved = {}
        for name, val in self.__dict__.items():
            moved[name] = val.to(device) if isinstance(val, torch.Tensor) else val
        return PagedWorkload(**moved)

    def clone_pools(self) -> "PagedWorkload":
        return replace(self, k_cache=self.k_cache.clone(), v_cache=self.v_cache.clone())

    def with_mask(self, *, is_cross_attention: bool, sliding_window_size: int) -> "PagedWorkload":
        return replace(self, is_cross_attention=is_cross_attention,
                       sliding_window_size=sliding_window_size)

    def select(self, reqs: List[int]) -> "PagedWorkload":
        """The same workload restricted to a subset of its requests (pools shared)."""
        kv_ip = self.kv_indptr.tolist()
        idx = torch.cat([self.kv_indices[kv_ip[b]:kv_ip[b + 1]] for b in reqs])
        kv_lens = [self.kv_lens[b] for b in reqs]
        ext = [self.extend_lens[b] for b in reqs]
        if self.kind == "decode":
            q = self.q[reqs]
            return replace(self, kv_lens=kv_lens, extend_lens=ext, q=q,
                           kv_indptr=_indptr(kv_lens), kv_indices=idx,
                           num_kv_splits=self.num_kv_splits[reqs])
        qo_ip = self.qo_indptr.tolist()
        rows = torch.cat([torch.arange(qo_ip[b], qo_ip[b + 1]) for b in reqs])
        return replace(
            self, kv_lens=kv_lens, extend_lens=ext, q=self.q[rows], kv_indptr=_indptr(kv_lens),
            kv_indices=idx, qo_indptr=_indptr(ext), prefix_lens=self.prefix_lens[reqs],
            max_len_extend=max(ext),
            new_k=None if self.new_k is None else self.new_k[rows],
            new_v=None if self.new_v is None else self.new_v[rows],
            out_loc=None if self.out_loc is None else self.out_loc[rows])

    # ---- algorithmic work -----------------------------------------------------------
    def attention_bytes(self) -> int:
        return roofline.attention_bytes(self.prefixes, self.extend_lens, self.kv_lens, self.n_q,
                                        self.n_kv, self.head_dim, self.is_cross_attention,
                                        self.sliding_window_size)

    def attention_flops(self) -> int:
        return roofline.attention_flops(self.prefixes, self.extend_lens, self.kv_lens, self.n_q,
                                        self.head_dim, self.is_cross_attention,
                                        self.sliding_window_size)

    def store_bytes(self) -> int:
        n = 0 if self.out_loc is None else int(self.out_loc.numel())
        return roofline.store_bytes(n, self.n_kv, self.head_dim)


def _indptr(lens) -> torch.Tensor:
    return torch.cumsum(torch.tensor([0] + list(lens), dtype=torch.int64), 0).to(torch.int32)


def _randn_bf16(shape, g: torch.Generator, device=None) -> torch.Tensor:
    """fp32 N(0,1) rounded to bf16, drawn in slabs so the fp32 temporary stays small.

    With a non-CPU ``device`` the values are drawn there, from a generator seeded by the next
    draw of ``g`` (multi-GiB pools take a minute on host cores); the stream of values then
    differs from the CPU one but is still a function of the seed alone.
    """
    device = torch.device(device) if device is not None else torch.device("cpu")
    gen = g
    if device.type != "cpu":
        gen = torch.Generator(device=device)
        gen.manual_seed(int(torch.randint(0, 2**31 - 1, (1,), generator=g)))
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(-1)
    step = 1 << 26
    for s in range(0, flat.numel(), step):
        n = min(step, flat.numel() - s)
        flat[s:s + n] = torch.randn(n, generator=gen, dtype=torch.float32,
                                    device=device).to(torch.bfloat16)
    return out


def _split_hint(kv_lens) -> torch.Tensor:
    return torch.tensor([min(MAX_KV_SPLITS, max(1, (l + 127) // 128)) for l in kv_lens],
                        dtype=torch.int32)


def build_workload(name: str, kind: str, *, seed: int, n_q: int, n_kv: int, head_dim: int = 128,
                   page_size: int = 16, kv_lens: List[int], extend_lens: Optional[List[int]] = None,
                   pool_pages: Optional[int] = None, pool_factor: float = 1.0,
                   store_new: bool = False, is_cross_attention: bool = False,
                   sliding_window_size: int = 0,
                   generator: Optional[torch.Generator] = None,
                   pool_device=None) -> PagedWorkload:
    g = generator if generator is not None else torch.Generator().manual_seed(seed)
    batch = len(kv_lens)
    if extend_lens is None:
        extend_lens = [1] * batch
    pages_per_req = [(l + page_size - 1) // page_size for l in kv_lens]
    used_pages = sum(pages_per_req)
    if pool_pages is None:
        pool_pages = max(1, int(math.ceil(used_pages * pool_factor)))
    assert pool_pages >= used_pages, "pool smaller than the pages the requests need"
    perm = torch.randperm(pool_pages, generator=g)
    offs = torch.arange(page_size, dtype=torch.int64)
    pieces, cur = [], 0
    for l, npg in zip(kv_lens, pages_per_req):
        pages = perm[cur:cur + npg]
        cur += npg
        slots = (pages[:, None] * page_size + offs[None, :]).reshape(-1)[:l]
        pieces.append(slots)
    kv_indices = (torch.cat(pieces) if pieces else torch.zeros(0, dtype=torch.int64)).to(torch.int32)
    kv_indptr = _indptr(kv_lens)
    num_slots = pool_pages * page_size
    k_cache = _randn_bf16((num_slots, n_kv, head_dim), g, pool_device)
    v_cache = _randn_bf16((num_slots, n_kv, head_dim), g, pool_device)
    total_q = sum(extend_lens)
    q = _randn_bf16((total_q, n_q, head_dim), g)
    wl = PagedWorkload(
        name=name, kind=kind, n_q=n_q, n_kv=n_kv, head_dim=head_dim, page_size=page_size,
        sm_scale=1.0 / math.sqrt(head_dim), kv_lens=list(kv_lens), extend_lens=list(extend_lens),
        q=q, k_cache=k_cache, v_cache=v_cache, kv_indptr=kv_indptr, kv_indices=kv_indices)
    if kind == "decode":
        wl.num_kv_splits = _split_hint(kv_lens)
    else:
        wl.qo_indptr = _indptr(extend_lens)
        wl.prefix_lens = torch.tensor([l - e for l, e in zip(kv_lens, extend_lens)],
                                      dtype=torch.int32)
        wl.max_len_extend = max(extend_lens) if extend_lens else 0
        wl.is_cross_attention = is_cross_attention
        wl.sliding_window_size = sliding_window_size
        if store_new:
            wl.new_k = _randn_bf16((total_q, n_kv, head_dim), g)
            wl.new_v = _randn_bf16((total_q, n_kv, head_dim), g)
            ip = kv_indptr.tolist()
            wl.out_loc = torch.cat([kv_indices[ip[b + 1] - extend_lens[b]:ip[b + 1]]
                                    for b in range(batch)]).to(torch.int32)
    return wl


def _randint_list(lo: int, hi: int, n: int, g: torch.Generator) -> List[int]:
    return torch.randint(lo, hi + 1, (n,), generator=g).tolist()


def _scaled(x: int, scale: float, floor: int = 1) -> int:
    return max(floor, int(round(x * scale)))


def config_workload(cfg: int, *, scale: float = 1.0, variant: str = "",
                    pool_device=None, head_dim: int = 128) -> PagedWorkload:
    """Workload of benchmark shape ``cfg`` (1..5); ``scale`` < 1 shrinks the lengths (and, for
    shape 3, the extend) for CPU-sized tests.  ``variant="window"`` selects the sliding
    window 1024 run of shape 5.  ``pool_device`` draws the two pools on that device.
    ``head_dim`` other than 128 (shape 3 only) gives the same extend at that head size."""
    g = torch.Generator().manual_seed(SEED_BASE + cfg)
    if head_dim != 128 and cfg != 3:
        raise ValueError("head_dim is selectable for shape 3 only")
    if cfg == 1:
        lens = [_scaled(l, scale) for l in (37, 128, 500, 1023)]
        return build_workload("cfg1_decode_qwen3_0.6b", "decode", seed=0, generator=g, n_q=16,
                              n_kv=8, kv_lens=lens, pool_pages=512, pool_device=pool_device)
    if cfg == 2:
        lens = _randint_list(_scaled(1024, scale), _scaled(8192, scale), 64, g)
        return build_workload("cfg2_decode_qwen3_8b", "decode", seed=0, generator=g, n_q=32,
                              n_kv=8, kv_lens=lens, pool_factor=1.5, pool_device=pool_device)
    if cfg == 3:
        ext = _scaled(512, scale)
        prefixes = _randint_list(0, _scaled(16384, scale), 8, g)
        name = "cfg3_extend_qwen3_8b" + ("" if head_dim == 128 else f"_head_dim_{head_dim}")
        return build_workload(name, "prefill", seed=0, generator=g, n_q=32, n_kv=8,
                              head_dim=head_dim, kv_lens=[p + ext for p in prefixes],
                              extend_lens=[ext] * 8, pool_factor=1.5, store_new=True,
                              pool_device=pool_device)
    if cfg == 4:
        lens = _randint_list(_scaled(32768, scale), _scaled(131072, scale), 16, g)
        return build_workload("cfg4_decode_qwen3_32b_long", "decode", seed=0, generator=g, n_q=64,
                              n_kv=8, kv_lens=lens, pool_factor=1.0, pool_device=pool_device)
    if cfg == 5:
        prefixes = _randint_list(_scaled(2048, scale), _scaled(8192, scale), 32, g)
        window = 0
        name = "cfg5_verify_full"
        if variant == "window":
            window = _scaled(1024, scale)
            name = "cfg5_verify_window"
        return build_workload(name, "prefill", seed=0, generator=g, n_q=32, n_kv=8,
                              kv_lens=[p + 8 for p in prefixes], extend_lens=[8] * 32,
                              pool_factor=1.0, sliding_window_size=window,
                              pool_device=pool_device)
    raise ValueError(f"unknown benchmark shape {cfg}")
