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
