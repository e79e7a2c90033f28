"""Seeded synthetic KV caches and block tables for the five benchmark configurations.

Shared by the parity tests and the benchmark so that both exercise the same
inputs. A *plane* is one layer's K (or V) cache: ``[blocks, *block_shape]``.
Plane ``(layer, kv)`` of a configuration is generated from its own seed
``base_seed * 10000 + layer * 2 + kv`` so that any plane can be regenerated alone
(the full caches are 8-80 GiB and are never mirrored on the host).

Nothing here calls the kernels; this is input generation only.
"""
from dataclasses import dataclass, replace
from typing import Tuple

import numpy as np
import torch


@dataclass(frozen=True)
class CacheConfig:
    name: str
    layers: int
    kv: int                     # planes per layer: 2 = separate K and V, 1 = single latent tensor
    block_shape: Tuple[int, ...]  # per-block shape, e.g. (16 tokens, 8 kv heads, 128 head dim)
    dtype: torch.dtype
    dev_blocks: int             # blocks per plane in the device cache
    host_blocks: int            # blocks per plane in the pinned host cache (0 = none)
    n_blocks: int               # blocks moved / gathered per launch
    dist: str                   # "normal", "uniform", "normal_half", "bytes"
    base_seed: int

    @property
    def planes(self):
        return self.layers * self.kv

    @property
    def block_elems(self):
        n = 1
        for s in self.block_shape:
            n *= s
        return n

    @property
    def elem_bytes(self):
        return torch.empty((), dtype=self.dtype).element_size()

    @property
    def block_bytes(self):
        return self.block_elems * self.elem_bytes

    @property
    def payload_bytes(self):
        """Bytes one launch moves in one direction: blocks x planes x block bytes."""
        return self.n_blocks * self.planes * self.block_bytes

    def scaled(self, layers=None, dev_blocks=None, host_blocks=None, n_blocks=None):
        """Same block geometry and dtype with fewer layers / blocks (CPU-sized parity cases)."""
        return replace(
            self,
            name=self.name + "-scaled",
            layers=self.layers if layers is None else layers,
            dev_blocks=self.dev_blocks if dev_blocks is None else dev_blocks,
            host_blocks=self.host_blocks if host_blocks is None else host_blocks,
            n_blocks=self.n_blocks if n_blocks is None else n_blocks,
        )


# The five configurations, in the order the benchmark definition lists them.
C1_GATHER_FP16 = CacheConfig("c1-gather-fp16", 1, 2, (16, 8, 128), torch.float16, 1024, 0, 32, "normal", 0)
C2_LLAMA8B_SWAP_OUT = CacheConfig("c2-llama3-8b-swap-out", 32, 2, (16, 8, 128), torch.bfloat16, 4096, 8192, 256,
                                  "normal", 2)
C3_LLAMA70B_SWAP_IN = CacheConfig("c3-llama3-70b-swap-in", 80, 2, (16, 8, 128), torch.bfloat16, 8192, 16384, 1024,
                                  "uniform", 3)
C4_MLA_ROUNDTRIP = CacheConfig("c4-mla-roundtrip", 61, 1, (64, 576), torch.bfloat16, 2048, 2048, 128,
                               "normal_half", 4)
C5_FP8_FRAGMENTED = CacheConfig("c5-fp8-fragmented", 32, 2, (16, 8, 128), torch.float8_e4m3fn, 8192, 8192, 4096,
                                "bytes", 5)

CONFIGS = {c.name: c for c in (C1_GATHER_FP16, C2_LLAMA8B_SWAP_OUT, C3_LLAMA70B_SWAP_IN, C4_MLA_ROUNDTRIP,
                               C5_FP8_FRAGMENTED)}


def plane_seed(cfg, layer, kv):
    return cfg.base_seed * 10000 + layer * 2 + kv


def _fill(shape, dist, dtype, gen, device):
    if dist == "bytes":
        raw = torch.randint(0, 256, shape, generator=gen, dtype=torch.uint8, device=device)
        return raw.view(dtype) if dtype != torch.uint8 else raw
    if dist == "uniform":
        return (torch.rand(shape, generator=gen, dtype=torch.float32, device=device) * 2 - 1).to(dtype)
    x = torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
    if dist == "normal_half":
        x = x * 0.5
    return x.to(dtype)


def make_plane(cfg, layer, kv, blocks, device="cpu"):
    """One plane ``[blocks, *block_shape]`` with the configuration's distribution.

    ``device="cpu"`` uses the CPU generator (the canonical data of the small parity
    cases); a CUDA device uses that device's generator with the same seed, which is
    how the multi-GiB full-size caches are filled without a host mirror. The two
    streams differ; tests always take expected values from the data actually
    generated, never from the seed.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(plane_seed(cfg, layer, kv))
    return _fill((blocks,) + tuple(cfg.block_shape), cfg.dist, cfg.dtype, gen, device)


def block_table(cfg, n=None, src_blocks=None, dst_blocks=None, seed_offset=0):
    """``(src_ids, dst_ids)``: n distinct random source blocks and n distinct destination slots."""
    n = cfg.n_blocks if n is None else n
    gen = torch.Generator()
    gen.manual_seed(cfg.base_seed * 10000 + 9000 + seed_offset)
    src = torch.randperm(src_blocks, generator=gen)[:n].contiguous()
    dst = torch.randperm(dst_blocks, generator=gen)[:n].contiguous()
    return src, dst


def pairs_tensor(src_ids, dst_ids):
    return torch.stack([src_ids.to(torch.int64), dst_ids.to(torch.int64)], dim=1).contiguous()


def gather_ids(cfg, n=None, blocks=None):
    """n block ids drawn uniformly without replacement (configuration 1)."""
    n = cfg.n_blocks if n is None else n
    blocks = cfg.dev_blocks if blocks is None else blocks
    gen = torch.Generator()
    gen.manual_seed(cfg.base_seed * 10000 + 9100)
    return torch.randperm(blocks, generator=gen)[:n].contiguous()


def fragmented_ids(total_blocks, n_ids, p=0.25, isolated_fraction=0.2, seed=5):
    """Block ids of a fragmented prefill (configuration 5): runs of consecutive blocks
    with lengths ~ Geometric(p) at uniformly drawn starts, mixed with isolated single
    blocks (about ``isolated_fraction`` of the ids), no block used twice. Runs are
    emitted in random order, so the gathered buffer alternates runs and singletons."""
    rs = np.random.RandomState(seed)
    if n_ids > total_blocks:
        raise ValueError("more ids than blocks")
    used = np.zeros(total_blocks, dtype=bool)
    pieces = []
    n_isolated = int(round(n_ids * isolated_fraction))
    remaining = n_ids - n_isolated
    guard = 0
    while remaining > 0 and guard < 100 * n_ids:
        guard += 1
        length = int(min(rs.geometric(p), remaining))
        start = int(rs.randint(0, total_blocks - length + 1))
        if used[start:start + length].any():
            continue
        used[start:start + length] = True
        pieces.append(np.arange(start, start + length, dtype=np.int64))
        remaining -= length
    free = np.flatnonzero(~used)
    if remaining > 0 or len(free) < n_isolated:
        # Dense tables: fall back to whatever is free, still without repeats.
        extra = rs.permutation(free)[:remaining + n_isolated]
        pieces.extend(np.array([b], dtype=np.int64) for b in extra)
    else:
        for b in rs.permutation(free)[:n_isolated]:
            pieces.append(np.array([b], dtype=np.int64))
    order = rs.permutation(len(pieces))
    ids = np.concatenate([pieces[i] for i in order]) if pieces else np.zeros(0, dtype=np.int64)
    assert len(ids) == n_ids and len(np.unique(ids)) == n_ids
    return torch.from_numpy(ids)


def as_bytes(t):
    """uint8 view ``[dim0, bytes_per_row]`` of a contiguous tensor (bit-exact comparisons)."""
    t = t.contiguous()
    return t.view(torch.uint8).reshape(t.shape[0], -1) if t.dim() > 1 else t.view(torch.uint8)
