"""Seeded synthetic inputs for the five benchmark configurations (C1..C5) of the fused
embedding path, and the algorithmic byte count used for the roofline.

All host randomness is ``numpy.random.Generator(PCG64)``: the feature list (rows, dim, mean bag
length, Zipf exponent) is drawn from ``default_rng(seed)``, feature ``f``'s bags and indices
from the ``f``-th child of ``SeedSequence(seed)``.  Tables are generated on the device with a
``torch.Generator`` seeded ``seed + f`` (mean 0, std 0.01), so a checker copies a table back
instead of regenerating it.

The reference's own datasets (``data_synthesis/data_generate.py``) are far smaller (tables of
at most 16 384 rows except mlperf, batches of at most 512); these configurations are the ones
this build is measured on.

====  ===  =====  ==========================  ===========================================
name  F    batch  tables                      bags / indices
====  ===  =====  ==========================  ===========================================
C1    4    512    100 000 x 32 fp32           exactly 4 lookups, uniform indices
C2    26   4096   10^U(3,7) x 64 fp32         exactly 1 lookup, Zipf(1.05)
C3    100  2048   10^U(3,6.7) x {8..128} f32  Poisson(m), m log-uniform [1,200], 5 % empty,
                                              Zipf(U(0.8,1.2))
C4    400  8192   10^U(4,7.3) x {16..256} f16 Poisson(m), m log-uniform [1,500], 5 % empty,
                                              Zipf(1.1)
C5    200  16384  10^U(4,7) x 128 int8        Poisson(m), m log-uniform [1,100], Zipf(1.05)
====  ===  =====  ==========================  ===========================================
"""

import math
from typing import List, NamedTuple, Optional, Sequence, Tuple

import numpy as np

TABLE_STD = 0.01
BASE_SEEDS = {"C1": 1001, "C2": 1002, "C3": 1003, "C4": 1004, "C5": 1005}


class FeatureSpec(NamedTuple):
    rows: int
    dim: int
    data_type: str      # "float" | "half" | "int8"
    mean_bag: float     # Poisson mean (or the exact length if fixed_len)
    fixed_len: bool     # every bag has exactly round(mean_bag) lookups
    empty_frac: float   # share of bags forced to length 0
    zipf_alpha: float   # 0 = uniform indices
    # > 0: bag lengths from a lognormal of mean mean_bag and this sigma of the logarithm instead
    # of a Poisson (a heavy tail: at 1.5 the longest of 2 048 bags is some hundred means long)
    len_sigma: float = 0.0
    # > 0: bag lengths from N(mean_bag, len_std) restricted to [0, len_max] (len_max 0 = no upper
    # end) and truncated to integers: the "multi-hot" families of the reference's data generator
    # (data_synthesis/data_generate.py:27-40)
    len_std: float = 0.0
    len_max: int = 0


class Workload(NamedTuple):
    name: str
    batch: int
    seed: int
    features: Tuple[FeatureSpec, ...]
    # "normal": N(0, 0.01) values.  "integer": small integers (fp32 / fp16) or integer bias and
    # power-of-two scale (int8), so that every sum is exact in fp32 whatever the order of the
    # additions and a checker can ask for identical bits.
    table_values: str = "normal"

    @property
    def num_features(self) -> int:
        return len(self.features)

    @property
    def embed_dim_sum(self) -> int:
        return sum(f.dim for f in self.features)

    def table_bytes(self) -> int:
        return sum(f.rows * row_stride(f.dim, f.data_type) for f in self.features)


def elem_bytes(data_type: str) -> int:
    return {"float": 4, "half": 2, "int8": 1}[data_type]


def row_stride(dim: int, data_type: str) -> int:
    if data_type == "int8":
        return (dim + 4 + 15) // 16 * 16
    return dim * elem_bytes(data_type)


def row_bytes(dim: int, data_type: str) -> int:
    """Algorithmic bytes per lookup: the payload, plus fp16 scale and bias for int8."""
    return dim * elem_bytes(data_type) + (4 if data_type == "int8" else 0)


def _log_uniform(rng: np.random.Generator, lo: float, hi: float, n: int) -> np.ndarray:
    return np.exp(rng.uniform(math.log(lo), math.log(hi), n))


# Models shaped like the reference's own example models (examples/models/A .. F there: 800 to
# 10 000 features, tables of 1 024 to 16 384 rows, dims 4 to 128, batches of at most 512): half
# the features one-hot, the rest "multi-hot" (truncated normal pooling factor), "multi-hot-static"
# (fixed pooling factor) and "multi-hot-one-side" (normal truncated at 0 only), in groups of like
# features.  Only these shape parameters are taken from there; every group's parameters, every
# table shape and every index is drawn here from the seed.
REF_SHAPED = {
    # name: (features, batch, seed, share of one-hot / multi-hot / static / one-side features)
    "REFA": (1000, 256, 2001, (0.50, 0.25, 0.15, 0.10)),
    "REFF4": (2500, 256, 2002, (0.50, 0.35, 0.15, 0.0)),
}
REF_GROUP = 50            # like features per group
REF_ZIPF_ALPHA = 1.05


def _table_rules():
    """TABLE_RULES / DIM_CHOICES of data_synthesis/table_config_generate.py (rows and the weighted
    choice of dims per feature family), loaded from that script."""
    import os
    from .utils import import_from_path
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    mod = import_from_path("table_config_generate",
                           os.path.join(root, "data_synthesis", "table_config_generate.py"))
    return mod.TABLE_RULES, mod.DIM_CHOICES


def make_ref_shaped(name: str, batch: Optional[int] = None, num_features: Optional[int] = None,
                    seed: Optional[int] = None) -> Workload:
    import random
    total, B, base_seed, shares = REF_SHAPED[name]
    total = num_features or total
    B = batch or B
    seed = base_seed if seed is None else seed
    rules, dim_choices = _table_rules()
    rng = np.random.default_rng(seed)
    dims_rng = random.Random(seed)
    kinds = ("one-hot", "multi-hot", "multi-hot-static", "multi-hot-one-side")
    counts = [int(round(total * share)) for share in shares]
    last = max(k for k, share in enumerate(shares) if share > 0)
    counts[last] = total - sum(c for k, c in enumerate(counts) if k != last)   # rounding
    feats: List[FeatureSpec] = []
    for kind, count in zip(kinds, counts):
        rows, weights = rules[kind]
        for g0 in range(0, count, REF_GROUP):
            n = min(REF_GROUP, count - g0)
            coverage = float(rng.choice([0.3, 0.5, 0.8, 1.0])) if kind != "one-hot" else 1.0
            mean = float(rng.choice([10, 50, 100, 200] if kind == "multi-hot-one-side" else [10, 50, 100]))
            std = mean * float(rng.choice([0.2, 0.5, 1.0]))
            top = int(mean * float(rng.choice([2, 5])))
            for dim in dims_rng.choices(dim_choices, weights, k=n):
                if kind == "one-hot":
                    spec = FeatureSpec(rows, dim, "float", 1.0, True, 1.0 - coverage, REF_ZIPF_ALPHA)
                elif kind == "multi-hot-static":
                    spec = FeatureSpec(rows, dim, "float", mean, True, 1.0 - coverage, REF_ZIPF_ALPHA)
                else:
                    spec = FeatureSpec(rows, dim, "float", mean, False, 1.0 - coverage, REF_ZIPF_ALPHA,
                                       len_std=std, len_max=top if kind == "multi-hot" else 0)
                feats.append(spec)
    return Workload(name, B, seed, tuple(feats))


def make_workload(name: str, batch: Optional[int] = None, num_features: Optional[int] = None,
                  max_rows: Optional[int] = None, seed: Optional[int] = None) -> Workload:
    """One of C1..C5, or one of the reference-shaped models REFA / REFF4.  ``batch`` /
    ``num_features`` / ``max_rows`` shrink the configuration (same distributions, smaller
    extents) for tests that must run in seconds."""
    name = name.upper()
    if name in REF_SHAPED:
        return make_ref_shaped(name, batch, num_features, seed)
    if name not in BASE_SEEDS:
        raise ValueError(f"unknown workload {name!r}; expected one of {sorted(BASE_SEEDS) + sorted(REF_SHAPED)}")
    seed = BASE_SEEDS[name] if seed is None else seed
    rng = np.random.default_rng(seed)

    def rows_draw(lo_exp: float, hi: float, n: int) -> np.ndarray:
        r = np.floor(10.0 ** rng.uniform(lo_exp, math.log10(hi), n)).astype(np.int64)
        return np.minimum(r, max_rows) if max_rows else r

    if name == "C1":
        F, B = num_features or 4, batch or 512
        rows = np.full(F, 100_000, dtype=np.int64)
        if max_rows:
            rows = np.minimum(rows, max_rows)
        feats = [FeatureSpec(int(r), 32, "float", 4.0, True, 0.0, 0.0) for r in rows]
    elif name == "C2":
        F, B = num_features or 26, batch or 4096
        rows = rows_draw(3, 1e7, F)
        feats = [FeatureSpec(int(r), 64, "float", 1.0, True, 0.0, 1.05) for r in rows]
    elif name == "C3":
        F, B = num_features or 100, batch or 2048
        rows = rows_draw(3, 5e6, F)
        dims = rng.choice([8, 16, 32, 64, 128], F)
        means = _log_uniform(rng, 1, 200, F)
        alphas = rng.uniform(0.8, 1.2, F)
        feats = [FeatureSpec(int(r), int(d), "float", float(m), False, 0.05, float(a))
                 for r, d, m, a in zip(rows, dims, means, alphas)]
    elif name == "C4":
        F, B = num_features or 400, batch or 8192
        rows = rows_draw(4, 2e7, F)
        dims = rng.choice([16, 32, 64, 128, 256], F)
        means = _log_uniform(rng, 1, 500, F)
        feats = [FeatureSpec(int(r), int(d), "half", float(m), False, 0.05, 1.1)
                 for r, d, m in zip(rows, dims, means)]
    else:  # C5
        F, B = num_features or 200, batch or 16384
        rows = rows_draw(4, 1e7, F)
        means = _log_uniform(rng, 1, 100, F)
        feats = [FeatureSpec(int(r), 128, "int8", float(m), False, 0.0, 1.05)
                 for r, m in zip(rows, means)]
    return Workload(name, B, seed, tuple(feats))


# ------------------------------------------------------------------------------------------------
# inputs
# ------------------------------------------------------------------------------------------------

def bounded_zipf(rng: np.random.Generator, alpha: float, support: int, n: int) -> np.ndarray:
    """Ranks in [1, support] with P(rank) ~ rank^-alpha (inverse CDF of the continuous
    approximation; valid for alpha <= 1 and huge supports, unlike ``numpy.random.zipf``)."""
    u = rng.random(n)
    if abs(alpha - 1.0) < 1e-9:
        rank = np.floor(float(support) ** u)
    else:
        e = 1.0 - alpha
        rank = np.floor(((float(support) ** e - 1.0) * u + 1.0) ** (1.0 / e))
    return np.clip(rank, 1, support).astype(np.int64)


def _affine_params(rng: np.random.Generator, support: int) -> Tuple[int, int]:
    """(a, b) with gcd(a, support) == 1, so rank -> (a*rank + b) % support is a permutation that
    scatters the hot ranks over the table."""
    if support <= 2:
        return 1, 0
    while True:
        a = int(rng.integers(1, support))
        if math.gcd(a, support) == 1:
            return a, int(rng.integers(0, support))


def gen_feature_inputs(spec: FeatureSpec, batch: int, seed_seq: np.random.SeedSequence
                       ) -> Tuple[np.ndarray, np.ndarray]:
    """(indices int32[L], offsets int32[batch + 1]) of one feature."""
    rng = np.random.Generator(np.random.PCG64(seed_seq))
    if spec.fixed_len:
        lens = np.full(batch, int(round(spec.mean_bag)), dtype=np.int64)
    elif spec.len_std > 0:
        hi = float(spec.len_max) if spec.len_max > 0 else np.inf
        lens = np.empty(batch, dtype=np.int64)
        filled = 0
        while filled < batch:               # rejection sampling of the truncated normal
            draw = rng.normal(spec.mean_bag, spec.len_std, max(2 * (batch - filled), 16))
            draw = draw[(draw >= 0) & (draw <= hi)]
            take = min(len(draw), batch - filled)
            lens[filled:filled + take] = draw[:take].astype(np.int64)
            filled += take
    elif spec.len_sigma > 0:
        mu = np.log(max(spec.mean_bag, 0.05)) - spec.len_sigma ** 2 / 2
        lens = np.floor(rng.lognormal(mu, spec.len_sigma, batch) + rng.random(batch)).astype(np.int64)
    else:
        lens = rng.poisson(spec.mean_bag, batch).astype(np.int64)
    if spec.empty_frac > 0:
        lens[rng.random(batch) < spec.empty_frac] = 0
    offsets = np.zeros(batch + 1, dtype=np.int64)
    np.cumsum(lens, out=offsets[1:])
    total = int(offsets[-1])
    if total >= 2 ** 31:
        raise ValueError("feature has more lookups than int32 offsets can address")
    if spec.zipf_alpha > 0:
        rank = bounded_zipf(rng, spec.zipf_alpha, spec.rows, total)
        a, b = _affine_params(rng, spec.rows)
        idx = (a * rank + b) % spec.rows      # a, rank < 2**31: no int64 overflow
    else:
        idx = rng.integers(0, spec.rows, total)
    return idx.astype(np.int32), offsets.astype(np.int32)


def gen_inputs(wl: Workload, workers: int = 0) -> Tuple[List[np.ndarray], List[np.ndarray]]:
    """Indices and offsets of every feature.  ``workers`` > 1 draws the features on that many
    threads (each feature has its own child seed, so the result does not depend on it)."""
    children = np.random.SeedSequence(wl.seed).spawn(wl.num_features)
    if workers > 1 and wl.num_features > 1:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=workers) as pool:
            pairs = list(pool.map(lambda sc: gen_feature_inputs(sc[0], wl.batch, sc[1]),
                                  zip(wl.features, children)))
    else:
        pairs = [gen_feature_inputs(spec, wl.batch, child) for spec, child in zip(wl.features, children)]
    return [p[0] for p in pairs], [p[1] for p in pairs]


def _integer_rows(spec: FeatureSpec, g, device, n: int):
    """``n`` rows of small integers (int8: integer codes, scale in {1/4, 1/2, 1, 2}, integer
    bias), for which every fp32 sum of a few thousand rows is exact in any order."""
    import torch
    from .quant import int8_row_stride
    if spec.data_type != "int8":
        w = torch.randint(-8, 9, (n, spec.dim), generator=g, device=device, dtype=torch.int32)
        return w.to(torch.float32 if spec.data_type == "float" else torch.float16)
    out = torch.zeros(n, int8_row_stride(spec.dim), dtype=torch.uint8, device=device)
    out[:, :spec.dim] = torch.randint(0, 256, (n, spec.dim), generator=g, device=device,
                                      dtype=torch.int32).to(torch.uint8)
    scale = torch.tensor([0.25, 0.5, 1.0, 2.0], device=device)[
        torch.randint(0, 4, (n,), generator=g, device=device)]
    bias = torch.randint(-8, 9, (n,), generator=g, device=device).float()
    sb = torch.stack([scale, bias], dim=1).half().contiguous()
    out[:, spec.dim:spec.dim + 4] = sb.view(torch.uint8).view(n, 4)
    return out


def gen_table(spec: FeatureSpec, seed: int, device, chunk_rows: int = 1 << 21,
              table_values: str = "normal"):
    """Device table of one feature: N(0, 0.01) fp32, rounded to fp16, or row-wise int8
    (``table_values="integer"``: small integers instead).  Filled in chunks of rows so that the
    temporaries stay small beside tables that nearly fill the device."""
    import torch
    from .quant import int8_row_stride, quantize_rowwise_int8
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if spec.data_type == "float":
        out = torch.empty(spec.rows, spec.dim, dtype=torch.float32, device=device)
    elif spec.data_type == "half":
        out = torch.empty(spec.rows, spec.dim, dtype=torch.float16, device=device)
    else:
        out = torch.empty(spec.rows, int8_row_stride(spec.dim), dtype=torch.uint8, device=device)
    for r0 in range(0, spec.rows, chunk_rows):
        r1 = min(spec.rows, r0 + chunk_rows)
        if table_values == "integer":
            out[r0:r1] = _integer_rows(spec, g, device, r1 - r0)
            continue
        w = torch.randn(r1 - r0, spec.dim, dtype=torch.float32, device=device, generator=g) * TABLE_STD
        if spec.data_type == "int8":
            out[r0:r1] = quantize_rowwise_int8(w)
        else:
            out[r0:r1] = w.to(out.dtype)
    return out


def gen_tables(wl: Workload, device) -> list:
    return [gen_table(spec, wl.seed + f, device, table_values=wl.table_values)
            for f, spec in enumerate(wl.features)]


# ------------------------------------------------------------------------------------------------
# roofline accounting
# ------------------------------------------------------------------------------------------------

def algorithmic_bytes(wl: Workload, num_lookups: Sequence[int]) -> int:
    """Bytes the path must move for one batch:
    sum_f [ L_f * (row_bytes_f + 4) + (batch + 1) * 4 + batch * dim_f * 4 ]
    (gathered rows + int32 indices + int32 offsets + fp32 output)."""
    total = 0
    for spec, L in zip(wl.features, num_lookups):
        total += int(L) * (row_bytes(spec.dim, spec.data_type) + 4)
        total += (wl.batch + 1) * 4 + wl.batch * spec.dim * 4
    return total


CACHE_LINE = 128       # bytes fetched from HBM at a time on an MI355X


def distinct_row_lines(indices: np.ndarray, stride: int, payload: int, line: int = CACHE_LINE) -> int:
    """Distinct ``line``-byte memory lines that hold the payload bytes of the rows ``indices``
    of a table whose rows are ``stride`` bytes apart (table base aligned to a line): narrow rows
    share lines, wide rows span several."""
    if len(indices) == 0:
        return 0
    rows = np.unique(np.asarray(indices, dtype=np.int64))
    first = rows * stride // line
    last = (rows * stride + payload - 1) // line
    # rows are sorted, so their line intervals are too: a row can only share its first line(s)
    # with the row before it
    prev_last = np.concatenate([[-1], last[:-1]])
    return int(np.maximum(last - np.maximum(first, prev_last + 1) + 1, 0).sum())


def compulsory_bytes(wl: Workload, indices: Sequence[np.ndarray], offsets: Sequence[np.ndarray],
                     line: int = CACHE_LINE) -> int:
    """Bytes that must cross the HBM pins for one batch even with perfect caches: every distinct
    memory line of the table rows the batch touches once, plus the index arrays, the offset
    arrays and the pooled output (each rounded up to whole lines).  Always at most
    ``algorithmic_bytes``, which counts a row as often as it is looked up."""
    def lines(nbytes: int) -> int:
        return -(-nbytes // line)
    total = 0
    for spec, idx, off in zip(wl.features, indices, offsets):
        used = idx[:int(off[-1])]
        total += distinct_row_lines(used, row_stride(spec.dim, spec.data_type),
                                    row_bytes(spec.dim, spec.data_type), line) * line
        total += lines(len(used) * 4) * line + lines(len(off) * 4) * line
    total += lines(wl.batch * wl.embed_dim_sum * 4) * line
    return total
