"""GPU: occupancy control of the fused kernel.  A library emitted for ``occ`` workgroups per CU
sizes its persistent grid ``CUs x occ`` and, when its registers and static LDS would let more
workgroups onto a CU, pads every workgroup with dynamic LDS so that ``occ`` fit and ``occ + 1``
do not (reference: get_max_concurrent_blocks / get_dyn_smem_size,
``RecFlex/sched_basic_csrc/include/utils.cuh:6-58``)."""

import numpy as np
import pytest

from helpers import oracle_output, require_lib

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,requested", [("c1_o2", 2), ("c1_o5", 5), ("c1", 4), ("fewbags", 8)])
def test_dynamic_lds_pad_pins_the_requested_occupancy(name, requested):
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.librecom import RecomLib
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    print(f"[case] occupancy pad: model={name} requested={requested}", flush=True)
    torch.cuda.init()
    lib = RecomLib(require_lib(name))
    assert lib.info.occupancy == requested
    li = lib.get_launch_info()
    assert li.compute_units == torch.cuda.get_device_properties(0).multi_processor_count
    assert li.lds_bytes_per_cu >= 64 * 1024 and li.num_vgprs > 0
    assert li.occupancy == requested
    assert lib.get_max_concurrent_blocks() == li.compute_units * requested
    per_wg = li.static_lds_bytes + li.dyn_lds_bytes
    if li.natural_occupancy > requested:
        assert li.dyn_lds_bytes > 0
        # `requested` workgroups fit into the LDS of a CU, one more does not
        assert requested * per_wg <= li.lds_bytes_per_cu < (requested + 1) * per_wg
    else:
        assert li.natural_occupancy == requested and li.dyn_lds_bytes == 0
    # what the registers allow: 512 per SIMD in blocks of 8, one wavefront of a 256-thread
    # workgroup per SIMD, at most 8
    regs = (li.num_vgprs + 7) // 8 * 8
    assert li.natural_occupancy <= min(8, 512 // regs)
    # the runtime's own answer for the padded launch, where it gives one, is not above the request
    assert li.padded_api_occupancy <= requested

    # and the padded library still computes the right thing on its full grid
    wl = prebuilt.model_spec(name).workload
    dev = torch.device("cuda", 0)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layer = FeatEmbed(dev, embed_tables=tables, librecom=lib)
    out = layer.forward_indices([torch.from_numpy(i).to(dev) for i in indices],
                                [torch.from_numpy(o).to(dev) for o in offsets]).cpu().numpy()
    want = oracle_output(wl, [t.cpu().numpy() for t in tables], indices, offsets)
    if wl.table_values == "integer":
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    else:
        assert np.allclose(out, want, rtol=1e-5, atol=1e-6)
