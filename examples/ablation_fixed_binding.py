"""Run-time thread binding against a binding frozen at emit time, on batches the frozen one was
not made for.

    python ablation_fixed_binding.py [--workload c3] [--steps 30]

The reference's ablation (``examples/run_fixed_thread.sh``, ``RecFlex/tuning/tuner.py:312-357``)
freezes the number of thread blocks per feature to the mean / max over the sampled batches and
compares kernel times on those same batches.  Here the two prebuilt libraries of the built-in
workload are compared: ``<workload>_tuned`` (every workgroup binds tiles to features from the
live offsets of the batch) and ``<workload>_tuned_static`` (the tile count per feature frozen to
what that binding chooses for the workload's own batch).  Both run the workload's batch, the same
batch cut to fewer samples, batches of the same features whose bags are two and four times as
long, and batches in which only every other feature's bags grow (the load moves between
features); outputs are compared bit for bit, and the fused kernel's duration is taken from HIP events
attached to its dispatch.  Prints one line per batch and a JSON summary.
"""

import argparse
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def kernel_us(layer, bound, out, steps: int) -> float:
    import torch
    from recflex_amd.hip_helper import HipEvent
    for _ in range(5):
        layer.forward_indices(bound, out=out)
    pairs = [(HipEvent(), HipEvent()) for _ in range(steps)]
    for pair in pairs:
        layer.forward_indices(bound, out=out, kernel_events=pair)
    torch.cuda.synchronize()
    return float(np.median([a.elapsed_us(b) for a, b in pairs]))


def longer_bags(indices, offsets, factors):
    """The same bags, each bag's lookups repeated ``factors[f]`` times (same rows, that many
    times the length); an int applies to every feature."""
    if isinstance(factors, int):
        factors = [factors] * len(indices)
    new_idx, new_off = [], []
    for idx, off, factor in zip(indices, offsets, factors):
        lens = np.diff(off).astype(np.int64)
        rep = lens * factor
        bag_of = np.repeat(np.arange(len(lens)), rep)
        k = np.arange(int(rep.sum()), dtype=np.int64) - np.repeat(np.cumsum(rep) - rep, rep)
        new_idx.append(idx[off[:-1].astype(np.int64)[bag_of] + k % lens[bag_of]].astype(np.int32))
        new_off.append(np.concatenate(([0], np.cumsum(rep))).astype(np.int32))
    return new_idx, new_off


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--workload", default="c3")
    parser.add_argument("--steps", type=int, default=30)
    args = parser.parse_args()

    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    names = (f"{args.workload}_tuned", f"{args.workload}_tuned_static")
    libs = []
    for name in names:
        path = prebuilt.lib_path(name)
        if not os.path.exists(path):
            sys.exit(f"{path} is not built: python -c 'from recflex_amd import prebuilt; prebuilt.build(\"{name}\")'")
        libs.append(path)
    wl = prebuilt.model_spec(names[0]).workload
    dev = torch.device("cuda", 0)
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    layers = [FeatEmbed(dev, embed_tables=tables, librecom=p) for p in libs]
    assert layers[0].lib.info.static_binding == 0 and layers[1].lib.info.static_binding == 1

    cases = [(f"the batch it was frozen for ({wl.batch} samples)", indices, offsets)]
    b = wl.batch
    while b > 64:
        b //= 4
        cases.append((f"first {b} samples",
                      [i[:o[b]] for i, o in zip(indices, offsets)], [o[:b + 1] for o in offsets]))
    for factor in (2, 4):
        i2, o2 = longer_bags(indices, offsets, factor)
        cases.append((f"{wl.batch} samples, bags {factor} x as long", i2, o2))

    # the load moves between features: every other feature's bags grow, the rest stay
    for factor in (4, 8):
        i2, o2 = longer_bags(indices, offsets, [factor if f % 2 == 0 else 1 for f in range(wl.num_features)])
        cases.append((f"{wl.batch} samples, every other feature's bags {factor} x", i2, o2))

    rows = []
    for label, idx, off in cases:
        d_idx = [torch.from_numpy(np.ascontiguousarray(i)).to(dev) for i in idx]
        d_off = [torch.from_numpy(np.ascontiguousarray(o)).to(dev) for o in off]
        batch = len(off[0]) - 1
        outs, times = [], []
        for layer in layers:
            bound = layer.bind_inputs(d_idx, d_off)
            out = torch.empty(batch * wl.embed_dim_sum, dtype=torch.float32, device=dev)
            times.append(kernel_us(layer, bound, out, args.steps))
            outs.append(out)
        same = bool(torch.equal(outs[0].view(torch.int32), outs[1].view(torch.int32)))
        rows.append({"batch": label, "lookups": int(sum(len(i) for i in idx)),
                     "run_time_binding_us": times[0], "frozen_binding_us": times[1],
                     "frozen_over_run_time": times[1] / times[0], "identical_bits": same})
        print(f"{label:52s} run-time binding {times[0]:9.2f} us   frozen {times[1]:9.2f} us   "
              f"x{times[1] / times[0]:.2f}   identical bits: {same}", flush=True)
    print(json.dumps({"workload": args.workload, "cases": rows}))


if __name__ == "__main__":
    main()
