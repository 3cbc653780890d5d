"""Seeded synthetic workloads: the five benchmark configurations of this path.

Metadata (table sizes, types, bag lengths, indices, per-sample weights) comes
from ``numpy.random.Generator(PCG64(1000 + config))`` on the host, so it is
identical wherever it is generated. Table bytes are drawn on the device the
problem is built on (torch generator, same seed) because the large
configurations hold tens to hundreds of GB; a checker that needs the bytes on
the host copies the tables it looks at back.

Index distribution after the reference's request generator
(fbgemm_gpu/fbgemm_gpu/tbe/utils/requests.py:319-372): z ~ Zipf(alpha),
(z - 1) mod rows, then a seeded permutation of the row ids.
"""
from dataclasses import dataclass, field

import numpy as np
import torch

FP32, FP16, INT8, INT4, INT2, BF16 = 0, 1, 2, 3, 4, 5
POOL_SUM, POOL_MEAN = 0, 1
_BITS = {FP32: 32, FP16: 16, BF16: 16, INT8: 8, INT4: 4, INT2: 2}


def unpadded_row_bytes(D, ty, sb=4):
    return {FP32: D * 4, FP16: D * 2, BF16: D * 2, INT8: D + sb, INT4: D // 2 + sb, INT2: D // 4 + sb}[ty]


def padded_row_bytes(D, ty, align, sb=4):
    r = unpadded_row_bytes(D, ty, sb)
    return (r + align - 1) // align * align


def zipf_indices(rng, alpha, rows, n):
    z = rng.zipf(alpha, size=n)
    base = (z - 1) % rows
    perm = rng.permutation(rows)
    return perm[base].astype(np.int64)


@dataclass
class TbeProblem:
    """Inputs of one table-batched forward, in the operator's own terms."""
    name: str
    T: int
    B: int
    Ds: np.ndarray
    tys: np.ndarray
    rows: np.ndarray
    row_bytes: np.ndarray
    row_alignment: int
    weights_offsets: np.ndarray  # int64 [T]
    D_offsets: np.ndarray        # int32 [T+1]
    dev_weights: torch.Tensor    # uint8, on `device`
    indices: torch.Tensor
    offsets: torch.Tensor
    indice_weights: torch.Tensor  # or None
    pooling_mode: int
    output_dtype: int
    lengths: np.ndarray          # host copy, [T*B]
    host_indices: np.ndarray
    host_offsets: np.ndarray
    host_weights: np.ndarray = None
    extra: dict = field(default_factory=dict)

    @property
    def total_D(self):
        return int(self.D_offsets[-1])

    @property
    def lookups(self):
        return int(self.host_offsets[-1])

    @property
    def physical_indices(self):
        """Row ids after the pruned-row remap (the indices themselves when no table is pruned)."""
        return self.extra.get("host_dense", self.host_indices)

    def kept_per_table(self):
        """Lookups that actually read a row (physical index != -1), per table."""
        kept = np.zeros(self.T, np.int64)
        phys = self.physical_indices
        for t in range(self.T):
            s, e = self.host_offsets[t * self.B], self.host_offsets[(t + 1) * self.B]
            kept[t] = int((phys[s:e] != -1).sum())
        return kept

    def useful_row_bytes(self):
        """The figure the roofline uses: unpadded row bytes (data + scale/bias) of
        every lookup that reads a row. Padding, indices, offsets, per-sample
        weights and output traffic are not credited."""
        kept = self.kept_per_table()
        return int(sum(int(k) * unpadded_row_bytes(int(D), int(ty)) for k, D, ty in zip(kept, self.Ds, self.tys)))

    def other_bytes(self):
        isz = self.indices.element_size()
        out_sz = 4 if self.output_dtype == FP32 else 2
        return {
            "indices": self.lookups * isz,
            "offsets": (self.T * self.B + 1) * isz,
            "per_sample_weights": self.lookups * 4 if self.indice_weights is not None else 0,
            "output": self.B * self.total_D * out_sz,
            "remap_entries": self.lookups * 4 if "remap" in self.extra else 0,
        }

    def table_host_bytes(self, t):
        """uint8 copy of table t's rows on the host."""
        s = int(self.weights_offsets[t])
        n = int(self.rows[t]) * int(self.row_bytes[t])
        return self.dev_weights[s:s + n].cpu().numpy()


def _fill_table(buf, rows, row_bytes, D, ty, gen, scale_range, chunk_rows=1 << 20):
    """Random rows in the TBE layout (fp16 scale, fp16 bias, then data), in place."""
    dev = buf.device
    view = buf.view(rows, row_bytes)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        n = r1 - r0
        if ty in (INT8, INT4, INT2):
            view[r0:r1] = torch.randint(0, 256, (n, row_bytes), dtype=torch.uint8, device=dev, generator=gen)
            hdr = torch.empty(n, 2, dtype=torch.float32, device=dev)
            hdr[:, 0].uniform_(scale_range[0], scale_range[1], generator=gen)
            hdr[:, 1].uniform_(-1.0, 1.0, generator=gen)
            view[r0:r1, :4] = hdr.to(torch.float16).view(torch.uint8)
        elif ty == FP16:
            vals = torch.empty(n, D, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0, generator=gen)
            view[r0:r1, :2 * D] = vals.to(torch.float16).view(torch.uint8)
            if row_bytes > 2 * D:
                view[r0:r1, 2 * D:] = 0
        else:
            vals = torch.empty(n, D, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0, generator=gen)
            view[r0:r1, :4 * D] = vals.view(torch.uint8)
            if row_bytes > 4 * D:
                view[r0:r1, 4 * D:] = 0


def build_tbe(name, seed, specs, B, lengths_fn, alpha, weighted, pooling_mode, output_dtype,
              device, row_alignment=16, index_dtype=np.int64, scale_ranges=None, prune_frac=0.0,
              pruned_keep=None):
    """specs: list of (rows, D, ty). lengths_fn(rng, n) -> bag lengths. With
    ``pruned_keep`` = p, rows are LOGICAL rows: each table keeps a row with
    probability p, stores only the kept rows, and indices are logical ids that
    an int32 mapping (-1 = pruned) turns into physical rows."""
    rng = np.random.default_rng(np.random.PCG64(seed))
    T = len(specs)
    rows = np.array([s[0] for s in specs], np.int64)
    logical = rows.copy()
    mappings = []
    if pruned_keep is not None:
        for t in range(T):
            keep = rng.random(int(logical[t])) < pruned_keep
            m = np.full(int(logical[t]), -1, np.int32)
            m[keep] = np.arange(int(keep.sum()), dtype=np.int32)
            mappings.append(m)
            rows[t] = max(1, int(keep.sum()))
    Ds = np.array([s[1] for s in specs], np.int32)
    tys = np.array([s[2] for s in specs], np.uint8)
    row_bytes = np.array([padded_row_bytes(int(D), int(ty), row_alignment) for D, ty in zip(Ds, tys)], np.int64)
    sizes = (rows * row_bytes + 127) // 128 * 128  # each table starts on a 128-byte boundary
    weights_offsets = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int64)
    total = int(sizes.sum())
    D_offsets = np.concatenate([[0], np.cumsum(Ds)]).astype(np.int32)

    lengths = lengths_fn(rng, T * B).astype(np.int64)
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(index_dtype)
    idx_parts = []
    for t in range(T):
        n = int(offsets[(t + 1) * B] - offsets[t * B])
        part = zipf_indices(rng, alpha, int(logical[t]), n)
        if prune_frac > 0:
            part[rng.random(n) < prune_frac] = -1
        idx_parts.append(part)
    indices = np.concatenate(idx_parts).astype(index_dtype) if idx_parts else np.zeros(0, index_dtype)
    w = rng.uniform(0.0, 1.0, size=len(indices)).astype(np.float32) if weighted else None

    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    dev_weights = torch.zeros(total, dtype=torch.uint8, device=device)
    for t in range(T):
        s = int(weights_offsets[t])
        n = int(rows[t] * row_bytes[t])
        sr = (0.01, 0.1) if int(tys[t]) != INT8 else (0.001, 0.01)
        if scale_ranges:
            sr = scale_ranges.get(int(tys[t]), sr)
        _fill_table(dev_weights[s:s + n], int(rows[t]), int(row_bytes[t]), int(Ds[t]), int(tys[t]), gen, sr)

    extra = {}
    if mappings:
        remap_offsets = np.concatenate([[0], np.cumsum(logical)]).astype(np.int64)
        remap = np.concatenate(mappings)
        dense = indices.copy()
        for t in range(T):
            s, e = int(offsets[t * B]), int(offsets[(t + 1) * B])
            dense[s:e] = mappings[t][indices[s:e]]
        extra = {"remap": torch.from_numpy(remap).to(device), "remap_offsets": torch.from_numpy(remap_offsets).to(device),
                 "host_remap": remap, "host_remap_offsets": remap_offsets, "host_dense": dense}

    return TbeProblem(
        extra=extra,
        name=name, T=T, B=B, Ds=Ds, tys=tys, rows=rows, row_bytes=row_bytes,
        row_alignment=row_alignment, weights_offsets=weights_offsets, D_offsets=D_offsets,
        dev_weights=dev_weights, indices=torch.from_numpy(indices).to(device),
        offsets=torch.from_numpy(offsets).to(device),
        indice_weights=None if w is None else torch.from_numpy(w).to(device),
        pooling_mode=pooling_mode, output_dtype=output_dtype, lengths=lengths,
        host_indices=indices, host_offsets=offsets, host_weights=w)


def config3(device, scale=1.0, rows_scale=None, only_type=None):
    """64 tables, int4/int8/fp16 = 50/25/25 %, rows 10**U[5,7], D in {64,128,256}, B = 2048 per
    table, L = min(Poisson(30), 200), Zipf(1.1), fp32 per-sample weights, weighted sum, fp16 out."""
    seed = 1003
    rng = np.random.default_rng(np.random.PCG64(seed + 7919))
    T = 64
    tys = rng.choice([INT4, INT8, FP16], size=T, p=[0.5, 0.25, 0.25])
    rows = np.round(10 ** rng.uniform(5, 7, size=T)).astype(np.int64)
    Ds = rng.choice([64, 128, 256], size=T)
    if only_type is not None:  # experiment: same shapes, one row type
        tys = np.full(T, only_type)
    rows_scale = scale if rows_scale is None else rows_scale
    if rows_scale != 1.0:
        rows = np.maximum(64, (rows * rows_scale).astype(np.int64))
    B = max(4, int(round(2048 * scale)))
    specs = [(int(r), int(d), int(t)) for r, d, t in zip(rows, Ds, tys)]
    return build_tbe("config3: 64-table mixed int4/int8/fp16 TBE forward", seed, specs, B,
                     lambda g, n: np.minimum(g.poisson(30, size=n), 200), 1.1, True, POOL_SUM, FP16, device)


def config5(device, scale=1.0, tables_int4=400, tables_int2=32):
    """400 x 3,000,000 x 256 int4 + 32 x 1,000,000 x 32 int2, B = 16384 per table,
    L = Poisson(15), Zipf(1.2), sum pooling, bf16 out."""
    seed = 1005
    r4 = max(64, int(3_000_000 * scale))
    r2 = max(64, int(1_000_000 * scale))
    specs = [(r4, 256, INT4)] * tables_int4 + [(r2, 32, INT2)] * tables_int2
    B = max(4, int(round(16384 * scale)))
    return build_tbe("config5: HBM-sized int4 + int2 TBE forward", seed, specs, B,
                     lambda g, n: g.poisson(15, size=n), 1.2, False, POOL_SUM, BF16, device)


def config4_batched(device, scale=1.0, tables=32):
    """Config 4 as ONE table-batched call: 32 pruned int4 tables (2,000,000 logical rows x 64,
    half of them pruned) in the operator's layout with 4-byte row alignment (36-byte rows), B =
    4096, L = U{5..50}, Zipf(1.05) over logical ids, mean pooling, fp32 out; the int32 mappings of
    all tables concatenated as pruned_array_lookup takes them."""
    seed = 1004
    logical = max(64, int(2_000_000 * scale))
    B = max(4, int(round(4096 * scale)))
    return build_tbe("config4: 32 pruned int4 tables, remap fused into one table-batched forward", seed,
                     [(logical, 64, INT4)] * tables, B, lambda g, n: g.integers(5, 51, size=n), 1.05, False,
                     POOL_MEAN, FP32, device, row_alignment=4, pruned_keep=0.5)


@dataclass
class SpmdmProblem:
    """Inputs of one single-table pooled lookup (trailer layout)."""
    name: str
    ty: int
    D: int
    rows: int            # physical rows
    data_size: int       # what indices are checked against (logical rows when pruned)
    table: torch.Tensor  # uint8
    indices: torch.Tensor
    offsets: torch.Tensor
    weights: torch.Tensor
    remap: torch.Tensor
    normalize: bool
    out_ty: int
    host_indices: np.ndarray
    host_offsets: np.ndarray
    host_remap: np.ndarray = None

    @property
    def num_bags(self):
        return len(self.host_offsets) - 1

    @property
    def lookups(self):
        return int(self.host_offsets[-1])

    def row_bytes(self):
        sb = 8 if self.ty == INT8 else 4
        return (self.D * _BITS[self.ty] + 7) // 8 + sb

    def useful_row_bytes(self):
        if self.host_remap is None:
            kept = self.lookups
        else:
            kept = int((self.host_remap[self.host_indices] != -1).sum())
        return kept * self.row_bytes()


def _trailer_table(device, gen, ty, rows, D, scale_range):
    pb = (D * _BITS[ty] + 7) // 8
    sb = 8 if ty == INT8 else 4
    t = torch.randint(0, 256, (rows, pb + sb), dtype=torch.uint8, device=device, generator=gen)
    hdr = torch.empty(rows, 2, dtype=torch.float32, device=device)
    hdr[:, 0].uniform_(scale_range[0], scale_range[1], generator=gen)
    hdr[:, 1].uniform_(-1.0, 1.0, generator=gen)
    t[:, pb:] = (hdr if ty == INT8 else hdr.to(torch.float16)).view(torch.uint8)
    return t.reshape(-1)


def config1(device, scale=1.0):
    """100,000 x 128 fused 8-bit rows (fp32 scale/bias trailer), 1024 bags x 20, uniform int64
    indices, int32 offsets, sum, fp32 out."""
    seed = 1001
    rng = np.random.default_rng(np.random.PCG64(seed))
    rows, D, nb, L = max(64, int(100_000 * scale)), 128, max(4, int(1024 * scale)), 20
    idx = rng.integers(0, rows, size=nb * L).astype(np.int64)
    off = (np.arange(nb + 1) * L).astype(np.int32)
    gen = torch.Generator(device=device); gen.manual_seed(seed)
    table = _trailer_table(device, gen, INT8, rows, D, (1e-3, 1e-2))
    return SpmdmProblem("config1: single-table fused 8-bit", INT8, D, rows, rows, table,
                        torch.from_numpy(idx).to(device), torch.from_numpy(off).to(device), None, None,
                        False, FP32, idx, off)


def config2(device, scale=1.0):
    """4,000,000 x 128 int4 rows (fp16 scale/bias trailer), 4096 bags, L = U{1..40}, Zipf(1.05)
    int64 indices with a seeded permutation, int32 offsets, sum, fp16 out."""
    seed = 1002
    rng = np.random.default_rng(np.random.PCG64(seed))
    rows, D, nb = max(64, int(4_000_000 * scale)), 128, max(4, int(4096 * scale))
    lens = rng.integers(1, 41, size=nb)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    idx = zipf_indices(rng, 1.05, rows, int(off[-1]))
    gen = torch.Generator(device=device); gen.manual_seed(seed)
    table = _trailer_table(device, gen, INT4, rows, D, (0.01, 0.1))
    return SpmdmProblem("config2: single-table int4", INT4, D, rows, rows, table,
                        torch.from_numpy(idx).to(device), torch.from_numpy(off).to(device), None, None,
                        False, FP16, idx, off)


def config4(device, scale=1.0, tables=32):
    """32 pruned int4 tables: 2,000,000 logical rows x 64, half of the rows mapped to -1 by an
    int32 table, B = 4096, L = U{5..50}, Zipf(1.05) over logical ids, mean pooling, fp32 out.
    Returns one SpmdmProblem per table (the row-wise-sparse kernel is a per-table call)."""
    seed = 1004
    rng = np.random.default_rng(np.random.PCG64(seed))
    logical, D, nb = max(64, int(2_000_000 * scale)), 64, max(4, int(4096 * scale))
    gen = torch.Generator(device=device); gen.manual_seed(seed)
    probs = []
    for t in range(tables):
        keep = rng.random(logical) >= 0.5
        mapping = np.full(logical, -1, np.int32)
        mapping[keep] = np.arange(int(keep.sum()), dtype=np.int32)
        rows = max(1, int(keep.sum()))
        lens = rng.integers(5, 51, size=nb)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        idx = zipf_indices(rng, 1.05, logical, int(off[-1]))
        table = _trailer_table(device, gen, INT4, rows, D, (0.01, 0.1))
        probs.append(SpmdmProblem(
            f"config4[{t}]: pruned int4", INT4, D, rows, logical, table,
            torch.from_numpy(idx).to(device), torch.from_numpy(off).to(device), None,
            torch.from_numpy(mapping).to(device), True, FP32, idx, off, mapping))
    return probs
