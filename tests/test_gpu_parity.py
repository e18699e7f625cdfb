"""GPU parity: the HIP fused kernel, called through the C ABI of a prebuilt librecom.so, against
the CPU oracle on identical seeded inputs."""

import numpy as np
import pytest

from helpers import check_against_oracle, oracle_output, require_lib

pytestmark = pytest.mark.gpu


def _run_model(name: str, form: str = "pointers", tile_bytes: int = 0, grid_blocks: int = 0,
               xcd_segments: int = 0):
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.host import RecomHost
    from recflex_amd.workloads import gen_inputs, gen_tables

    spec = prebuilt.model_spec(name)
    wl = spec.workload
    dev = torch.device("cuda", 0)
    print(f"[case] model={name} form={form} F={wl.num_features} B={wl.batch} "
          f"tile_bytes={tile_bytes} grid={grid_blocks} xcd_segments={xcd_segments}", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    if form == "pointers":
        d_idx = [torch.from_numpy(i).to(dev) for i in indices]
        d_off = [torch.from_numpy(o).to(dev) for o in offsets]
        out = layer.forward_indices(d_idx, d_off, tile_bytes=tile_bytes, grid_blocks=grid_blocks,
                                    xcd_segments=xcd_segments)
    else:
        packed, byte_offsets = RecomHost().pack(offsets, indices)
        out = layer(torch.from_numpy(packed).to(dev), torch.from_numpy(byte_offsets).to(dev),
                    output_size=wl.batch * wl.embed_dim_sum * 4, tile_bytes=tile_bytes,
                    grid_blocks=grid_blocks).view(wl.batch, wl.embed_dim_sum)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    host_tables = [t.cpu().numpy() for t in tables]
    want = oracle_output(wl, host_tables, indices, offsets)
    return wl, got, want


def _assert_parity(wl, got, want):
    assert got.shape == want.shape == (wl.batch, wl.embed_dim_sum)
    failures = check_against_oracle(wl, got, want)
    msg = "\n".join(f"feature {f} {spec}: max_abs={a:.3e} max_rel={r:.3e}" for f, spec, a, r in failures[:10])
    assert not failures, f"{len(failures)} features out of tolerance\n{msg}"


@pytest.mark.parametrize("name", ["c1", "edge", "variants", "c2s", "c3s", "c3s_bind_once", "c4s", "c5s"])
def test_model_matches_oracle(name):
    _assert_parity(*_run_model(name))


@pytest.mark.parametrize("name", ["c1", "c3s"])
def test_packed_buffer_form(name):
    _assert_parity(*_run_model(name, form="packed"))


@pytest.mark.parametrize("tile_bytes,grid,xcd", [(4096, 0, 0), (1 << 20, 0, 0), (0, 1, 0), (0, 7, 0),
                                                 (16384, 3, 0), (0, 0, -1), (0, 0, 1), (4096, 0, 16),
                                                 (0, 5, 2), (0, 1024, 1000)])
def test_binding_is_result_invariant(tile_bytes, grid, xcd):
    """Any tile size / grid size / tile walk must give the same pooled output (only the binding
    changes); grids that are not a multiple of the 8 XCDs and more segments than tiles included."""
    _assert_parity(*_run_model("c3s", tile_bytes=tile_bytes, grid_blocks=grid, xcd_segments=xcd))


@pytest.mark.parametrize("name", ["c3s_drawn_all", "c3s_ordered"])
@pytest.mark.parametrize("tile_bytes,grid,xcd", [(4096, 0, 0), (1 << 20, 0, 0), (0, 1, 0), (0, 7, 0),
                                                 (16384, 96, -1), (0, 0, 1), (4096, 0, 128),
                                                 (0, 1024, 1000), (0, 8, 3)])
def test_drawn_walks_are_result_invariant(name, tile_bytes, grid, xcd):
    """The same for libraries whose tiles are drawn from ticket counters (all of them; the last
    two passes of an ordered tile space): one workgroup, grids that are not a multiple of the
    8 XCDs (one counter for the device), more segments than tiles, fewer tiles than workgroups."""
    wl, got, want = _run_model(name, tile_bytes=tile_bytes, grid_blocks=grid, xcd_segments=xcd)
    assert wl.table_values == "integer"
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("name", ["variants", "edge", "onehots", "wide", "wider", "widest", "longbags"])
def test_integer_tables_are_bit_exact(name):
    """Integer-valued tables make every fp32 sum exact, so each schedule variant (any lane
    split, any reduction tree) must reproduce the oracle's bits."""
    wl, got, want = _run_model(name)
    assert wl.table_values == "integer"
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("tile_bytes,grid,xcd", [(4096, 0, 0), (65536, 0, 0), (1 << 20, 0, 0),
                                                 (1 << 24, 0, 0), (16384, 1, 0), (16384, 96, 0),
                                                 (32768, 300, -1), (8192, 0, 16)])
def test_split_bags_are_bit_exact_under_any_binding(tile_bytes, grid, xcd):
    """Bags of thousands of lookups summed by several workgroups each.  How many follows from
    the tile size and the grid (a part is a quarter of a workgroup's share of the batch, at
    least a tile and 256 KiB): 12 for the longest bags on the full grid, 3 with 1 MiB tiles,
    none with 16 MiB tiles or on a single workgroup.  Any tile walk.
    Integer-valued tables: bit for bit."""
    wl, got, want = _run_model("longbags", tile_bytes=tile_bytes, grid_blocks=grid, xcd_segments=xcd)
    assert wl.table_values == "integer"
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("batch", [1, 5, 40, 300, 2500])
def test_split_bags_on_other_batches_and_repeated_launches(batch):
    """The split-bag library on batches of other sizes (parts per bag: at most what 2048 slots
    allow, 64 at 5 bags, 6 at 300, none at 2500), bag lengths from empty to 9000 within one
    feature, a single bag of 40 000 lookups among empty ones (64 parts on a fp32 D=128 table),
    three launches in a row on the same workspace (the arrival counters must be back at zero
    after each).  Integer-valued tables: bit for bit."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_tables

    wl = prebuilt.model_spec("longbags").workload
    dev = torch.device("cuda", 0)
    print(f"[case] longbags on a ragged batch: B={batch}", flush=True)
    rng = np.random.default_rng(500 + batch)
    tables = gen_tables(wl, dev)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("longbags"))
    assert layer.workspace is not None
    host_tables = [t.cpu().numpy() for t in tables]
    scale = max(1, batch // 40)            # keeps the larger batches to a few million lookups
    for launch in range(3):
        indices, offsets = [], []
        for f, spec in enumerate(wl.features):
            kind = (f + launch) % 4
            if kind == 0:
                lens = rng.integers(0, 9000 // scale + 2, batch)
            elif kind == 1:
                lens = np.full(batch, 3000 // scale + 1) * (rng.random(batch) < 0.7)
            elif kind == 2:
                lens = np.zeros(batch, dtype=np.int64)
                # int8 sums stay exact in fp32 up to some ten thousand rows
                lens[rng.integers(0, batch)] = 8191 if spec.data_type == "int8" else 40000
            else:
                lens = rng.integers(0, 6, batch)
            off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            indices.append(rng.integers(0, spec.rows, int(off[-1])).astype(np.int32))
            offsets.append(off)
        d_idx = [torch.from_numpy(i).to(dev) for i in indices]
        d_off = [torch.from_numpy(o).to(dev) for o in offsets]
        got = layer.forward_indices(d_idx, d_off, tile_bytes=16384 if launch == 1 else 0).cpu().numpy()
        want = oracle_output(wl._replace(batch=batch), host_tables, indices, offsets)
        assert got.shape == want.shape == (batch, wl.embed_dim_sum)
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, f"launch {launch}: {len(bad)} elements differ, first at {bad[:5].tolist()}"
    # every arrival counter is back at zero: the counters follow each feature's 2048 * D slots
    ws = layer.workspace.cpu().numpy()
    pos = 0
    for spec in wl.features:
        pos += 2048 * spec.dim
        assert not ws[pos:pos + 2048].any(), f"arrival counters of a D={spec.dim} feature not reset"
        pos += 2048


def test_split_bags_give_the_same_bits_on_every_launch():
    """Whichever workgroup of a bag finishes last adds the partial sums in part order, so the
    output does not depend on the order of arrival: sixty launches with N(0, 0.01) tables (where
    any other order of the additions would show) under changing tile walks (the grid stays: it
    decides into how many parts a bag is split), all identical to the first, bit for bit."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec("longbags").workload._replace(table_values="normal")
    dev = torch.device("cuda", 0)
    print(f"[case] longbags launched sixty times: B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("longbags"))
    first = layer.forward_indices(d_idx, d_off, tile_bytes=32768).clone()
    out = torch.empty_like(first)
    for k in range(60):
        out.fill_(float("nan"))
        layer.forward_indices(d_idx, d_off, out=out, tile_bytes=32768,
                              xcd_segments=(0, -1, 1, 16, 4, 64)[k % 6])
        assert torch.equal(out.view(torch.int32), first.view(torch.int32)), f"launch {k}"


def test_split_bags_match_the_oracle_on_normal_tables():
    """fp32 / fp16 / int8 tables of N(0, 0.01) values, bags of thousands of lookups split over
    workgroups: a tree of partial sums against the oracle's sequential sum.  Sums of this
    length differ between any two orders by more than the 1e-5 asserted on the benchmark
    configurations (bags <= 500), so the relative bound here is 1e-4 for fp32 tables and the
    1e-3 of the fp16 / int8 path otherwise, measured against the largest magnitude of the
    feature's output."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec("longbags").workload._replace(table_values="normal")
    dev = torch.device("cuda", 0)
    print(f"[case] longbags with normal tables: B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("longbags"))
    got = layer.forward_indices([torch.from_numpy(i).to(dev) for i in indices],
                                [torch.from_numpy(o).to(dev) for o in offsets]).cpu().numpy()
    want = oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets)
    col = 0
    for spec in wl.features:
        g, w = got[:, col:col + spec.dim], want[:, col:col + spec.dim]
        bound = (1e-4 if spec.data_type == "float" else 1e-3) * np.abs(w).max() + 1e-6
        assert np.abs(g - w).max() <= bound, (spec, float(np.abs(g - w).max()), float(bound))
        col += spec.dim


@pytest.mark.parametrize("name", ["b128", "b512"])
def test_other_workgroup_sizes_are_bit_exact(name):
    """Libraries emitted for 128 and 512 threads per workgroup (2 and 8 wavefronts): every
    template and element type, integer-valued tables, identical bits."""
    wl, got, want = _run_model(name)
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


def test_onehot_is_bit_exact():
    """Bags of exactly one lookup are a row copy: identical bits (C2 shape, shrunk)."""
    wl, got, want = _run_model("c2s")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("case", ["one_each", "as_many_lookups_as_bags", "zero_or_one", "ragged",
                                  "one_long_among_ones", "all_empty"])
@pytest.mark.parametrize("batch", [1, 77, 1024])
def test_row_copy_template_on_any_input(case, batch):
    """``rfx::onehot_bags`` (``OneHotBagSchedule``, 28 candidates over fp32 / fp16 / int8 rows) on
    inputs it is and is not meant for: exactly one lookup per bag (the hint holds: an index is
    fetched together with its bag's offsets); as many lookups as bags but lengths 2, 0, 1, ...
    (the hint is set and wrong); bags of zero or one lookup (no hint); empty bags beside bags of
    2 to 100 lookups (the pass goes to the team routine with a per-wavefront stage slice); one
    bag of 500 lookups among bags of one (handed on to a whole wavefront); no lookup at all.
    Integer-valued tables: bit for bit, for every element type (row copy, scale and bias,
    staged output)."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_tables

    wl = prebuilt.model_spec("onehots").workload
    assert wl.table_values == "integer" and wl.num_features <= 512      # the hint is live
    dev = torch.device("cuda", 0)
    print(f"[case] onehots, {case}, B={batch}", flush=True)
    rng = np.random.default_rng(batch * 31 + len(case))
    tables = gen_tables(wl, dev)
    indices, offsets = [], []
    for f, spec in enumerate(wl.features):
        if case == "one_each":
            lens = np.ones(batch, dtype=np.int64)
        elif case == "as_many_lookups_as_bags":
            lens = np.ones(batch, dtype=np.int64)
            for b in range(f % 3, batch - 1, 3):           # 2, 0 in place of 1, 1
                lens[b], lens[b + 1] = 2, 0
        elif case == "zero_or_one":
            lens = (rng.random(batch) < 0.7).astype(np.int64)
        elif case == "ragged":
            lens = rng.integers(2, 101, batch) * (rng.random(batch) < 0.5)
        elif case == "one_long_among_ones":
            lens = np.ones(batch, dtype=np.int64)
            lens[rng.integers(0, batch)] = 500
        else:
            lens = np.zeros(batch, dtype=np.int64)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        if case == "as_many_lookups_as_bags":
            assert off[-1] == batch
        indices.append(rng.integers(0, spec.rows, int(off[-1])).astype(np.int32))
        offsets.append(off)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("onehots"))
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    got = layer.forward_indices(d_idx, d_off).cpu().numpy()
    want = oracle_output(wl._replace(batch=batch), [t.cpu().numpy() for t in tables], indices, offsets)
    assert got.shape == want.shape == (batch, wl.embed_dim_sum)
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("name", ["onehots", "c3s_outliers", "fewbags128"])
def test_lookup_count_hint_sizes_tiles_and_nothing_else(name):
    """``recom_process_args.d_lookup_counts``: the binding takes the lookups per feature from the
    caller instead of reading ``offsets[batch]`` of every feature.  Right figures (what
    ``bind_inputs`` passes), none, and wrong ones -- all zero, all equal to the batch (which tells
    the row-copy schedule that every bag has one lookup), ten times too many -- give the same
    output: bit for bit on integer-valued tables, also where the figures change how a split bag
    is cut into parts."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec(name).workload
    assert wl.table_values == "integer"
    dev = torch.device("cuda", 0)
    print(f"[case] {name}: lookup-count hint", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    bound = layer.bind_inputs([torch.from_numpy(i).to(dev) for i in indices],
                              [torch.from_numpy(o).to(dev) for o in offsets])
    assert bound.lookup_counts.cpu().tolist() == [len(i) for i in indices]
    want = oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets)
    true = bound.lookup_counts
    variants = {"right": true, "none": None, "zero": torch.zeros_like(true),
                "one_per_bag": torch.full_like(true, wl.batch), "tenfold": true * 10}
    for label, counts in variants.items():
        got = layer.forward_indices(bound._replace(lookup_counts=counts)).cpu().numpy()
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, f"{label}: {len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("name", ["c3s_ordered", "c3s_outliers_ordered", "wide_ordered", "wider_ordered",
                                  "onehots_ordered", "c3s_drawn_all", "wide_drawn_all_flat"])
def test_tile_order_and_drawn_end_change_no_bit(name):
    """A library emitted with ``tile_order`` numbers the features inside the kernel by their
    place in the tile space and finds what the caller passes per feature through a table; with
    ``drawn_tail`` the last passes of the walk are drawn from ticket counters.  Neither may
    change a bit of the output: random orders on a model that keeps its addresses in LDS (with
    split regions; with outlier tiles), one that reads them per tile, one bound once per launch,
    the row-copy template with every tile drawn, and two libraries emitted with every tile
    drawn (the first ticket asked for ahead of the binding), one of them on the flat walk with
    its single counter.  Three launches on one workspace (the
    ticket counters must be back at zero), with and without the lookup-count hint, also through
    the entry point that uses the library's static workspace.  Integer-valued tables: bit for
    bit against the oracle."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    spec = prebuilt.model_spec(name)
    wl = spec.workload
    assert wl.table_values == "integer"
    assert spec.emit_kwargs.get("tile_order") or spec.emit_kwargs.get("drawn_tail")
    dev = torch.device("cuda", 0)
    print(f"[case] {name}: F={wl.num_features} B={wl.batch} {sorted(k for k in spec.emit_kwargs)}", flush=True)
    tables = gen_tables(wl, dev)
    host_tables = [t.cpu().numpy() for t in tables]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    for launch in range(3):
        indices, offsets = gen_inputs(wl._replace(seed=wl.seed + 31 * launch))
        bound = layer.bind_inputs([torch.from_numpy(i).to(dev) for i in indices],
                                  [torch.from_numpy(o).to(dev) for o in offsets])
        if launch == 1:
            bound = bound._replace(lookup_counts=None)
        got = layer.forward_indices(bound).cpu().numpy()
        want = oracle_output(wl, host_tables, indices, offsets)
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, f"launch {launch}: {len(bad)} elements differ, first at {bad[:5].tolist()}"
    if layer.lib.info.static_workspace and layer.lib.workspace_bytes:
        out = torch.full((wl.batch * wl.embed_dim_sum,), float("nan"), device=dev)
        for _ in range(2):
            layer.lib.process(layer.embed_table_ptrs.data_ptr(), out.data_ptr(), wl.batch,
                              io_ptrs=bound.io_ptrs.data_ptr(), static_workspace=True,
                              stream=torch.cuda.current_stream(dev).cuda_stream)
        torch.cuda.synchronize()
        got = out.cpu().numpy().reshape(want.shape)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_gather_probe_runs():
    """The measurement aid of bench.py: fetches the rows of a batch and nothing else.  It must
    run to completion on ragged inputs (empty features, rows of 1 to 64 vectors) and take time."""
    import torch
    from recflex_amd import prebuilt
    from benchaid.gather_probe import GatherProbe
    from recflex_amd.workloads import gen_inputs, gen_tables, row_stride

    wl = prebuilt.model_spec("edge").workload
    dev = torch.device("cuda", 0)
    print(f"[case] gather probe on edge: F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    indices, _ = gen_inputs(wl)
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    probe = GatherProbe(dev, tables, d_idx, [row_stride(f.dim, f.data_type) for f in wl.features])
    strides = [row_stride(f.dim, f.data_type) for f in wl.features]
    assert probe.n_chunks == sum(-(-len(i) // 1024) for i, s in zip(indices, strides) if s >= 16)
    for kwargs in ({"in_flight": 2}, {"in_flight": 8, "segments": 16}, {"workgroups_per_cu": 3, "segments": 2}):
        assert probe.time_us(steps=3, warmup=1, **kwargs) > 0
    best = probe.best_time_us(steps=2)
    assert best["us"] > 0 and best["in_flight"] in (2, 4, 8)
    # with an output-sized buffer to fill: every byte of it is written, nothing beyond it
    # (what is written are sums of raw table bits read as floats, possibly NaN: compare bits)
    mark = 0x4B1D4B1D
    buf = torch.full((wl.batch * wl.embed_dim_sum + 8,), mark, dtype=torch.int32, device=dev)
    assert probe.time_with_output_us(best, buf[4:-4].view(torch.float32), steps=2) > 0
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert (host[:4] == mark).all() and (host[-4:] == mark).all() and (host[4:-4] != mark).all()


def test_pending_error_of_an_unrelated_call_does_not_fail_the_launch():
    """recom_process reports its own launch: an error that an earlier, unrelated HIP call left in
    the thread's last-error slot (here the profiler gate a ROCm 7 runtime refuses) is not its."""
    import ctypes
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.hip_helper import HipProfiler
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec("c1").workload
    dev = torch.device("cuda", 0)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("c1"))
    out = layer.forward_indices(d_idx, d_off).clone()
    want = oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets)
    out.zero_()
    torch.cuda.synchronize()

    hip = ctypes.CDLL("libamdhip64.so")
    rc = hip.hipProfilerStart()                      # 801 on ROCm 7; 0 where the gate exists
    print(f"[case] hipProfilerStart() -> {rc}, then a c1 launch into a preallocated output", flush=True)
    layer.forward_indices(d_idx, d_off, out=out)     # allocates nothing, must not see that error
    hip.hipGetLastError()                            # hand torch a clean slot
    torch.cuda.synchronize()
    _assert_parity(wl, out.cpu().numpy(), want)

    prof = HipProfiler()
    prof.start()
    prof.stop()                      # accepted whether the runtime implements the gates or not
    assert not torch.isnan(torch.empty(4, device=dev).fill_(1.0)).any()    # nothing left pending


@pytest.mark.parametrize("batch,seed", [(1, 0), (3, 1), (64, 2), (257, 3), (1000, 4)])
def test_every_schedule_variant_on_ragged_batches(batch, seed):
    """The 161-variant library (every template, lane split and element type) on batches it was
    not built around: any batch size, bag lengths with a heavy tail, runs of empty bags, features
    without a single lookup.  Integer-valued tables, so the comparison is bit for bit."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_tables

    wl = prebuilt.model_spec("variants").workload
    assert wl.table_values == "integer"
    dev = torch.device("cuda", 0)
    print(f"[case] variants on a ragged batch: B={batch} seed={seed}", flush=True)
    rng = np.random.default_rng(1000 + seed)
    tables = gen_tables(wl, dev)
    indices, offsets = [], []
    for f, spec in enumerate(wl.features):
        kind = (f + seed) % 5
        if kind == 0:
            lens = np.zeros(batch, dtype=np.int64)                        # no lookup at all
        elif kind == 1:
            lens = rng.geometric(0.08, batch) * (rng.random(batch) < 0.6)  # heavy tail, 40 % empty
        elif kind == 2:
            lens = np.zeros(batch, dtype=np.int64)
            lens[rng.integers(0, batch)] = 3000       # one outlier: summed by a whole wavefront
        elif kind == 3:
            lens = rng.integers(0, 4, batch)
        else:
            lens = np.full(batch, 1 + f % 9)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        indices.append(rng.integers(0, spec.rows, int(off[-1])).astype(np.int32))
        offsets.append(off)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("variants"))
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    got = layer.forward_indices(d_idx, d_off).cpu().numpy()
    shrunk = wl._replace(batch=batch)
    want = oracle_output(shrunk, [t.cpu().numpy() for t in tables], indices, offsets)
    assert got.shape == want.shape == (batch, wl.embed_dim_sum)
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.parametrize("name", ["c3s", "wider", "longbags", "c3s_outliers", "c3s_drawn_all"])
def test_launch_replays_inside_a_hip_graph(name):
    """recom_process is a single kernel launch on the caller's stream (binding happens on the
    device, no host-side task mapping, no copies), so a serving loop can capture it once and
    replay it (a library bound once per launch -- by default above 3 072 features -- launches its binding kernel first: two
    kernel nodes; a library whose tiles are drawn leaves its ticket counters at zero for the next
    replay).  Captured after one eager call; replayed four times, each time with new bag
    lengths and lookups written into the same index / offset buffers, with eager work and
    synchronisations in between; every replay is compared bit for bit with an eager launch."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec(name).workload
    dev = torch.device("cuda", 0)
    print(f"[case] {name} captured in a graph: F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    batches = [gen_inputs(wl._replace(seed=wl.seed + 31 * k)) for k in range(4)]
    capacity = [max(len(b[0][f]) for b in batches) for f in range(wl.num_features)]
    d_idx = [torch.zeros(max(1, c), dtype=torch.int32, device=dev) for c in capacity]
    d_off = [torch.zeros(wl.batch + 1, dtype=torch.int32, device=dev) for _ in range(wl.num_features)]
    out = torch.empty(wl.batch, wl.embed_dim_sum, dtype=torch.float32, device=dev)
    eager_out = torch.empty_like(out)

    def load(batch):
        indices, offsets = batch
        for f in range(wl.num_features):
            d_idx[f][:len(indices[f])].copy_(torch.from_numpy(indices[f]))
            d_off[f].copy_(torch.from_numpy(offsets[f]))

    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    load(batches[0])
    layer.forward_indices(d_idx, d_off, out=eager_out)       # first call: launch state, addresses
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.forward_indices(d_idx, d_off, out=out)

    for k in (1, 2, 3, 0):
        load(batches[k])
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        layer.forward_indices(d_idx, d_off, out=eager_out)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), eager_out.view(torch.int32)), f"replay of batch {k}"
        want = oracle_output(wl, [t.cpu().numpy() for t in tables], *batches[k])
        _assert_parity(wl, got.cpu().numpy(), want)


def test_check_inputs_names_what_a_launch_would_trip_over():
    """FeatEmbed.check_inputs accepts the generated batch and refuses, without launching
    anything, offsets that decrease or overrun the index array and indices outside the table."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec("c1").workload
    dev = torch.device("cuda", 0)
    print("[case] check_inputs on c1", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("c1"))
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    layer.check_inputs(d_idx, d_off)

    def broken(which, f, pos, value):
        idx, off = [t.clone() for t in d_idx], [t.clone() for t in d_off]
        (idx if which == "idx" else off)[f][pos] = value
        return idx, off

    for args, what in ((("idx", 1, 7, wl.features[1].rows), "indices span"),
                       (("idx", 2, 0, -1), "indices span"),
                       (("off", 0, 5, 1 << 20), "offsets decrease"),
                       (("off", 3, wl.batch, len(indices[3]) + 1), "beyond"),
                       (("off", 0, 0, 1), "expected 0")):
        with pytest.raises(ValueError, match=what):
            layer.check_inputs(*broken(*args))


def test_bound_inputs_give_the_same_output():
    """bind_inputs validates the tensors and uploads their addresses once; calls with its result
    skip the per-feature host work and must launch exactly what the list form launches, also
    after the bound tensors were refilled in place."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import BoundInputs, FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec("c3s").workload
    dev = torch.device("cuda", 0)
    print(f"[case] c3s through bind_inputs: F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    first, second = gen_inputs(wl), gen_inputs(wl._replace(seed=wl.seed + 5))
    cap = [max(len(a), len(b), 1) for a, b in zip(first[0], second[0])]
    d_idx = [torch.zeros(c, dtype=torch.int32, device=dev) for c in cap]
    d_off = [torch.zeros(wl.batch + 1, dtype=torch.int32, device=dev) for _ in cap]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("c3s"))
    bound = layer.bind_inputs(d_idx, d_off)
    assert isinstance(bound, BoundInputs) and bound.batch == wl.batch
    for indices, offsets in (first, second):
        for f in range(wl.num_features):
            d_idx[f][:len(indices[f])].copy_(torch.from_numpy(indices[f]))
            d_off[f].copy_(torch.from_numpy(offsets[f]))
        got = layer.forward_indices(bound).cpu().numpy()
        same = layer.forward_indices(d_idx, d_off).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), same.view(np.uint32))
        _assert_parity(wl, got, oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets))
    with pytest.raises(TypeError):
        layer.bind_inputs([t.long() for t in d_idx], d_off)
    with pytest.raises(ValueError):
        layer.bind_inputs(d_idx[:-1], d_off[:-1])


def test_two_libraries_write_column_slabs_of_one_buffer():
    """output_row_stride: a model split by features over two libraries (or GPUs) writes each
    library's [batch, sum(dim)] block straight into its columns of the common output."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    dev = torch.device("cuda", 0)
    parts = []
    for name in ("c3s", "c5s"):
        wl = prebuilt.model_spec(name).workload._replace(batch=100)
        tables = gen_tables(wl, dev)
        indices, offsets = gen_inputs(wl)
        parts.append((name, wl, tables, indices, offsets))
    widths = [p[1].embed_dim_sum for p in parts]
    print(f"[case] slabs of {widths} columns in one [100, {sum(widths) + 8}] buffer", flush=True)
    whole = torch.full((100, sum(widths) + 8), float("nan"), dtype=torch.float32, device=dev)
    col = 4                                     # slabs need not start at column 0
    for (name, wl, tables, indices, offsets), width in zip(parts, widths):
        layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
        d_idx = [torch.from_numpy(i).to(dev) for i in indices]
        d_off = [torch.from_numpy(o).to(dev) for o in offsets]
        got = layer.forward_indices(d_idx, d_off, out=whole[:, col:col + width])
        assert got.data_ptr() == whole[:, col:col + width].data_ptr()
        col += width
    torch.cuda.synchronize()
    host = whole.cpu().numpy()
    assert np.isnan(host[:, :4]).all() and np.isnan(host[:, col:]).all()    # nothing outside the slabs
    col = 4
    for (name, wl, tables, indices, offsets), width in zip(parts, widths):
        want = oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets)
        _assert_parity(wl, np.ascontiguousarray(host[:, col:col + width]), want)
        col += width
    # a slab whose columns would break the kernel's 16-byte stores is refused
    from recflex_amd.librecom import RecomError
    name, wl, tables, indices, offsets = parts[0]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    with pytest.raises(RecomError):
        layer.forward_indices(d_idx, d_off, out=whole[:, 2:2 + widths[0]])


@pytest.mark.parametrize("name", ["c3s", "wider", "c3s_outliers"])
def test_kernel_events_take_the_dispatch_time_and_change_nothing(name):
    """``start_event`` / ``stop_event`` of the C ABI: the launch goes through
    ``hipExtLaunchKernel``, the output keeps its bits, and the pair reads a duration that is
    positive and no longer than a pair of event records around the same launch."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.hip_helper import HipEvent
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec(name).workload
    dev = torch.device("cuda", 0)
    print(f"[case] kernel events model={name} F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    bound = layer.bind_inputs([torch.from_numpy(i).to(dev) for i in indices],
                              [torch.from_numpy(o).to(dev) for o in offsets])
    plain = layer.forward_indices(bound).clone()
    torch.cuda.synchronize()
    inside, around = [], []
    for _ in range(5):
        pair = (HipEvent(), HipEvent())
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        timed = layer.forward_indices(bound, kernel_events=pair)
        e.record()
        torch.cuda.synchronize()
        assert torch.equal(timed.view(torch.int32), plain.view(torch.int32))
        inside.append(pair[0].elapsed_us(pair[1]))
        around.append(s.elapsed_time(e) * 1e3)
    print(f"   dispatch {min(inside):.2f} us, event records around it {min(around):.2f} us", flush=True)
    assert all(0.0 < t < 1e5 for t in inside)
    assert min(inside) <= min(around) * 1.05
