"""``recom_process_static_workspace`` -- the entry point for callers that cannot allocate device
memory -- against ``recom_process`` on the same inputs, both called through the C ABI (ctypes on
the prebuilt ``librecom.so``).  The two must give identical bits: same kernels, the workspace in
the library's static device array instead of the caller's buffer.  Two calls in a row on each
library, the second on a smaller batch (the array keeps what the first call left in it)."""

import ctypes

import numpy as np
import pytest

from helpers import require_lib

# (model, what its workspace holds)
CASES = [("longbags", "split-bag partial sums and arrival counters"),
         ("c3s_outliers", "split regions and the outlier list"),
         ("wider", "the once-per-launch binding table"),
         ("c1", "nothing")]


def test_static_workspace_limit_is_refused_without_a_device():
    """A library whose workspace is beyond the static array's maximum returns
    RECOM_ESTATIC_WORKSPACE before any HIP call; argument checks are those of recom_process."""
    from recflex_amd import prebuilt
    from recflex_amd.librecom import (RECOM_ESTATIC_WORKSPACE, RECOM_STATIC_WORKSPACE_MAX_BYTES,
                                      RecomLib, RecomProcessArgs)
    big = RecomLib(prebuilt.ensure_built("manysplit"))
    assert big.workspace_bytes > RECOM_STATIC_WORKSPACE_MAX_BYTES and big.info.static_workspace == 0
    ok = dict(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=4)
    assert big.lib.recom_process_static_workspace(ctypes.byref(RecomProcessArgs(**ok))) \
        == RECOM_ESTATIC_WORKSPACE
    assert big.lib.recom_process_static_workspace(None) == 1
    small = RecomLib(prebuilt.ensure_built("longbags"))
    assert 0 < small.workspace_bytes <= RECOM_STATIC_WORKSPACE_MAX_BYTES
    assert small.info.static_workspace == 1
    assert small.lib.recom_process_static_workspace(ctypes.byref(RecomProcessArgs(batch=-1))) == 1
    # an empty batch launches nothing and needs no workspace argument
    a = RecomProcessArgs(d_embed_table_ptrs=8, d_io_ptrs=8, d_output=16, batch=0)
    assert small.lib.recom_process_static_workspace(ctypes.byref(a)) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name,holds", CASES)
def test_static_workspace_matches_caller_workspace(name, holds):
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.librecom import RecomLib
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec(name).workload
    dev = torch.device("cuda", 0)
    lib = RecomLib(require_lib(name))
    assert lib.info.static_workspace == 1
    tables = gen_tables(wl, dev)
    table_ptrs = torch.tensor([t.data_ptr() for t in tables], dtype=torch.int64, device=dev)
    indices, offsets = gen_inputs(wl)
    caller_ws = torch.zeros(max(1, (lib.workspace_bytes + 3) // 4), dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    for call, batch in enumerate((wl.batch, max(1, wl.batch // 3))):
        print(f"[case] static workspace: model={name} ({holds}) call={call} batch={batch}", flush=True)
        # the first `batch` bags of every feature
        d_off = [torch.from_numpy(np.ascontiguousarray(o[:batch + 1])).to(dev) for o in offsets]
        d_idx = [torch.from_numpy(i).to(dev) for i in indices]
        flat = [0] * (2 * wl.num_features)
        flat[0::2] = [t.data_ptr() for t in d_idx]
        flat[1::2] = [t.data_ptr() for t in d_off]
        io_ptrs = torch.tensor(flat, dtype=torch.int64, device=dev)
        want = torch.full((batch, wl.embed_dim_sum), float("nan"), dtype=torch.float32, device=dev)
        got = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        lib.process(table_ptrs.data_ptr(), want.data_ptr(), batch, io_ptrs=io_ptrs.data_ptr(),
                    stream=stream, workspace=caller_ws.data_ptr(), workspace_bytes=caller_ws.numel() * 4)
        lib.process(table_ptrs.data_ptr(), got.data_ptr(), batch, io_ptrs=io_ptrs.data_ptr(),
                    stream=stream, static_workspace=True)
        torch.cuda.synchronize()
        w, g = want.cpu().numpy(), got.cpu().numpy()
        assert not np.isnan(w).any(), "recom_process left output elements unwritten"
        bad = np.argwhere(g.view(np.uint32) != w.view(np.uint32))
        assert bad.size == 0, f"call {call}: {len(bad)} elements differ, first at {bad[:5].tolist()}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["longbags", "c3s_outliers"])
def test_static_workspace_replays_inside_a_hip_graph(name):
    """The use the entry point is for: captured once (after one eager call on the device, which
    resolves the array's address and the launch state), replayed with new inputs in the same
    buffers, the program's own eager work and synchronisations between the replays; every replay
    has the bits of an eager ``recom_process`` on a caller workspace."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.librecom import RecomLib
    from recflex_amd.workloads import gen_inputs, gen_tables

    wl = prebuilt.model_spec(name).workload
    dev = torch.device("cuda", 0)
    lib = RecomLib(require_lib(name))
    assert lib.info.static_workspace == 1 and lib.workspace_bytes > 0
    print(f"[case] static workspace captured in a graph: model={name}", flush=True)
    tables = gen_tables(wl, dev)
    table_ptrs = torch.tensor([t.data_ptr() for t in tables], dtype=torch.int64, device=dev)
    batches = [gen_inputs(wl._replace(seed=wl.seed + 17 * k)) for k in range(3)]
    capacity = [max(len(b[0][f]) for b in batches) for f in range(wl.num_features)]
    d_idx = [torch.zeros(max(1, c), dtype=torch.int32, device=dev) for c in capacity]
    d_off = [torch.zeros(wl.batch + 1, dtype=torch.int32, device=dev) for _ in range(wl.num_features)]
    flat = [0] * (2 * wl.num_features)
    flat[0::2] = [t.data_ptr() for t in d_idx]
    flat[1::2] = [t.data_ptr() for t in d_off]
    io_ptrs = torch.tensor(flat, dtype=torch.int64, device=dev)
    caller_ws = torch.zeros(max(1, (lib.workspace_bytes + 3) // 4), dtype=torch.int32, device=dev)
    got = torch.empty(wl.batch, wl.embed_dim_sum, dtype=torch.float32, device=dev)
    want = torch.empty_like(got)

    def load(batch):
        indices, offsets = batch
        for f in range(wl.num_features):
            d_idx[f][:len(indices[f])].copy_(torch.from_numpy(indices[f]))
            d_off[f].copy_(torch.from_numpy(offsets[f]))

    def static_call():
        lib.process(table_ptrs.data_ptr(), got.data_ptr(), wl.batch, io_ptrs=io_ptrs.data_ptr(),
                    stream=torch.cuda.current_stream(dev).cuda_stream, static_workspace=True)

    load(batches[0])
    static_call()                                   # the eager call that must precede a capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    for k in (1, 2, 0, 1):
        load(batches[k])
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        lib.process(table_ptrs.data_ptr(), want.data_ptr(), wl.batch, io_ptrs=io_ptrs.data_ptr(),
                    stream=torch.cuda.current_stream(dev).cuda_stream, workspace=caller_ws.data_ptr(),
                    workspace_bytes=caller_ws.numel() * 4)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"replay of batch {k}"
