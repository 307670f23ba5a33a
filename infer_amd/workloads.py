"""Seeded synthetic inputs for the paged KV-cache path (decode step and prefill step).

The shapes are the ones the decode step of ``infer/engine/model_runner.py:110-126`` hands to
``infer/ops/attention.py:96-122``: new K/V rows ``[N, Hkv, D]``, caches ``[nblk, bs, Hkv, D]``,
``slot_mapping [N]`` int32, ``block_table [B, MB]`` int32 padded with -1, ``context_lens [B]``
int32 (lengths include the token appended this step).  Everything is bf16 and drawn from a CPU
``torch.Generator``, then moved to the requested device, so the same seed gives the same bits on the
CPU and on the GPU box; ``checksums`` hashes them (``tests/golden/workload_checksums.json`` holds the
values of the named configurations).  ``device_fill=True`` draws the cache contents on the device
instead: faster for the multi-gigabyte pools of a bandwidth sweep, but reproducible only per device,
so parity tests never use it.
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass, field

import torch


def checksums(wl) -> dict:
    """SHA-256 of the bytes of every tensor of a workload (on the host, C order), by field name."""
    out = {}
    for name, v in wl.__dict__.items():
        if isinstance(v, torch.Tensor):
            t = v.detach().cpu().contiguous()
            raw = t.view(torch.uint8) if t.numel() else t
            out[name] = hashlib.sha256(raw.numpy().tobytes() if t.numel() else b"").hexdigest()
    return out


@dataclass
class DecodeWorkload:
    name: str
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    scale: float
    q: torch.Tensor              # [B, Hq, D] bf16
    k_new: torch.Tensor          # [B, Hkv, D] bf16, the row appended this step
    v_new: torch.Tensor
    k_cache: torch.Tensor        # [nblk, bs, Hkv, D] bf16
    v_cache: torch.Tensor
    slot_mapping: torch.Tensor   # [B] int32
    block_table: torch.Tensor    # [B, MB] int32, -1 padded
    context_lens: torch.Tensor   # [B] int32
    lengths: list = field(default_factory=list)

    def to(self, device) -> "DecodeWorkload":
        moved = {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in self.__dict__.items()}
        return DecodeWorkload(**moved)

    @property
    def decode_bytes(self) -> int:
        return decode_algorithmic_bytes(self.lengths, self.num_q_heads, self.num_kv_heads,
                                        self.head_dim, self.block_size)

    @property
    def append_bytes(self) -> int:
        n = len(self.lengths)
        return append_algorithmic_bytes(n, n, self.num_kv_heads * self.head_dim)


def decode_algorithmic_bytes(lengths, hq, hkv, d, bs, itemsize=2) -> int:
    """Bytes one decode-attention launch must move: K and V of every live token once, Q in, O out,
    the used block-table entries and the length."""
    total = 0
    for n in lengths:
        total += 2 * n * hkv * d * itemsize + 2 * hq * d * itemsize + 4 * ((n + bs - 1) // bs) + 4
    return total


def append_algorithmic_bytes(n_rows, n_valid, dkv, itemsize=2) -> int:
    """Bytes one append launch must move: each valid K and V row read once and written once, plus
    the slot of every row."""
    return n_valid * 4 * dkv * itemsize + 4 * n_rows


def _tables(lengths, bs, nblk, gen):
    need = [(n + bs - 1) // bs for n in lengths]
    assert sum(need) <= nblk, "pool too small"
    perm = torch.randperm(nblk, generator=gen).tolist()
    tables, at = [], 0
    for c in need:
        tables.append(perm[at:at + c])
        at += c
    width = max(max(need), 1)
    padded = [t + [-1] * (width - len(t)) for t in tables]
    return tables, torch.tensor(padded, dtype=torch.int32)


def _draw_caches(shape, dgen, device, device_fill):
    if device_fill and str(device) != "cpu":
        g = torch.Generator(device=device).manual_seed(dgen.initial_seed())
        return (torch.randn(shape, generator=g, device=device, dtype=torch.bfloat16),
                torch.randn(shape, generator=g, device=device, dtype=torch.bfloat16))
    return (torch.randn(shape, generator=dgen, dtype=torch.bfloat16),
            torch.randn(shape, generator=dgen, dtype=torch.bfloat16))


def make_decode_workload(name, lengths, hq, hkv, d=128, bs=256, nblk=None, seed=0, q_scale=1.0,
                         pool_factor=1.2, device="cpu", device_fill=False) -> DecodeWorkload:
    """Build one decode step.  ``lengths`` include the token appended this step (so >= 1)."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    need = sum((n + bs - 1) // bs for n in lengths)
    if nblk is None:
        nblk = max(int(-(-need * pool_factor // 1)), need)
    tables, block_table = _tables(lengths, bs, nblk, gen)
    b = len(lengths)
    dgen = torch.Generator(device="cpu").manual_seed(seed + 1)
    k_cache, v_cache = _draw_caches((nblk, bs, hkv, d), dgen, device, device_fill)
    q = (torch.randn((b, hq, d), generator=dgen, dtype=torch.float32) * q_scale).to(torch.bfloat16)
    k_new = torch.randn((b, hkv, d), generator=dgen, dtype=torch.float32).to(torch.bfloat16)
    v_new = torch.randn((b, hkv, d), generator=dgen, dtype=torch.float32).to(torch.bfloat16)
    slots = [t[-1] * bs + (n - 1) % bs for n, t in zip(lengths, tables)]
    return DecodeWorkload(
        name=name, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, block_size=bs, scale=d ** -0.5,
        q=q, k_new=k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache,
        slot_mapping=torch.tensor(slots, dtype=torch.int32),
        block_table=block_table,
        context_lens=torch.tensor(lengths, dtype=torch.int32),
        lengths=list(lengths)).to(device)


def cfg1(device="cpu") -> DecodeWorkload:
    """Qwen3-0.6B-shaped decode step: 16/8 heads, batch 4, lengths {37, 256, 700, 1023}, 64 blocks."""
    return make_decode_workload("cfg1-qwen3-0.6b-b4", [37, 256, 700, 1023], 16, 8, nblk=64, seed=0,
                                device=device)


def cfg2_lengths(batch=64, lo=512, hi=4096, seed=0):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=gen).tolist()


def cfg2(device="cpu", batch=64, device_fill=False) -> DecodeWorkload:
    """Qwen3-8B-shaped decode step: 32/8 heads, batch 64, lengths U[512, 4096], pool 1.2x need,
    Q scaled by 1/sqrt(128)."""
    return make_decode_workload("cfg2-qwen3-8b-b64", cfg2_lengths(batch), 32, 8, seed=0,
                                q_scale=128 ** -0.5, device=device, device_fill=device_fill)


def cfg4(device="cpu", batch=8, ctx=32768, nblk=2048, device_fill=False) -> DecodeWorkload:
    """Qwen3-32B-shaped long-context decode: 64/8 heads, batch 8 x 32768 tokens, tables fully
    fragmented over a 2048-block pool."""
    return make_decode_workload("cfg4-qwen3-32b-b8-ctx32k", [ctx] * batch, 64, 8, nblk=nblk, seed=0,
                                device=device, device_fill=device_fill)


@dataclass
class PrefillWorkload:
    name: str
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    scale: float
    q: torch.Tensor              # [Tq, Hq, D]
    k_new: torch.Tensor          # [N, Hkv, D]  (N = Tq real rows + padding rows)
    v_new: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    slot_mapping: torch.Tensor   # [N] int32, -1 on padding rows
    row_of_query: torch.Tensor   # [Tq] int64: which row of k_new/v_new belongs to query token i
    block_table: torch.Tensor    # [nseq, MB] int32
    cu_seqlens_q: torch.Tensor
    cu_seqlens_k: torch.Tensor
    max_seqlen_q: int
    max_seqlen_k: int
    lengths: list = field(default_factory=list)
    cached: list = field(default_factory=list)

    def to(self, device) -> "PrefillWorkload":
        moved = {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in self.__dict__.items()}
        return PrefillWorkload(**moved)

    @property
    def append_bytes(self) -> int:
        n = int(self.slot_mapping.numel())
        valid = int((self.slot_mapping >= 0).sum())
        return append_algorithmic_bytes(n, valid, self.num_kv_heads * self.head_dim)


def make_prefill_workload(name, lengths, cached, hq, hkv, d=128, bs=256, seed=0, pad_fraction=0.05,
                          pool_factor=1.2, device="cpu") -> PrefillWorkload:
    """Varlen prefill step with prefix-cached blocks and ``-1`` padding rows mixed into the append.

    ``cached[i]`` (a multiple of ``bs``) tokens of sequence ``i`` are already in the cache; the
    other ``lengths[i] - cached[i]`` tokens are the queries and get appended.  ``pad_fraction``
    extra dummy rows with slot -1 are inserted at random places of the packed K/V rows.
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    need = sum((n + bs - 1) // bs for n in lengths)
    nblk = max(int(-(-need * pool_factor // 1)), need)
    tables, block_table = _tables(lengths, bs, nblk, gen)
    assert all(c % bs == 0 and c < n for c, n in zip(cached, lengths))
    cu_q, cu_k, slots = [0], [0], []
    for n, c, t in zip(lengths, cached, tables):
        cu_q.append(cu_q[-1] + n - c)
        cu_k.append(cu_k[-1] + n)
        slots.extend(t[p // bs] * bs + p % bs for p in range(c, n))
    tq = cu_q[-1]
    n_pad = int(round(tq * pad_fraction))
    n_rows = tq + n_pad
    is_pad = torch.zeros(n_rows, dtype=torch.bool)
    if n_pad:
        is_pad[torch.randperm(n_rows, generator=gen)[:n_pad]] = True
    row_of_query = torch.nonzero(~is_pad).flatten()
    slot_mapping = torch.full((n_rows,), -1, dtype=torch.int32)
    slot_mapping[row_of_query] = torch.tensor(slots, dtype=torch.int32)
    dgen = torch.Generator(device="cpu").manual_seed(seed + 1)
    k_cache, v_cache = _draw_caches((nblk, bs, hkv, d), dgen, device, False)
    q = torch.randn((tq, hq, d), generator=dgen, dtype=torch.float32).to(torch.bfloat16)
    k_new = torch.randn((n_rows, hkv, d), generator=dgen, dtype=torch.float32).to(torch.bfloat16)
    v_new = torch.randn((n_rows, hkv, d), generator=dgen, dtype=torch.float32).to(torch.bfloat16)
    return PrefillWorkload(
        name=name, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, block_size=bs, scale=d ** -0.5,
        q=q, k_new=k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache,
        slot_mapping=slot_mapping, row_of_query=row_of_query, block_table=block_table,
        cu_seqlens_q=torch.tensor(cu_q, dtype=torch.int32),
        cu_seqlens_k=torch.tensor(cu_k, dtype=torch.int32),
        max_seqlen_q=max(n - c for n, c in zip(lengths, cached)), max_seqlen_k=max(lengths),
        lengths=list(lengths), cached=list(cached)).to(device)


def cfg3(device="cpu", nseq=16, lo=64, hi=2048, seed=0, hq=32, hkv=8) -> PrefillWorkload:
    """Qwen3-8B-shaped varlen prefill: 16 prompts U[64, 2048], 0-50 % of each already cached
    (rounded down to whole blocks), 5 % padding rows with slot -1."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    lengths = torch.randint(lo, hi + 1, (nseq,), generator=gen).tolist()
    frac = (torch.rand(nseq, generator=gen) * 0.5).tolist()
    cached = [int(f * n) // 256 * 256 for f, n in zip(frac, lengths)]
    return make_prefill_workload("cfg3-qwen3-8b-prefill16", lengths, cached, hq, hkv, seed=seed,
                                 device=device)
