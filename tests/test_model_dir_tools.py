"""CPU tests of the model-directory utilities beside tune.py: compress / decompress,
schedule_config_gen, table_config_generate (reference: examples/compress.py, examples/decompress.py,
examples/schedule_config_gen.py, data_synthesis/table_config_generate.py)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EX = os.path.join(ROOT, "examples")


def run(script, *args):
    subprocess.run([sys.executable, script, *args], check=True, cwd=ROOT)


def write(path, text):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(text)


def make_model(tmp_path):
    m = str(tmp_path / "model")
    write(f"{m}/data_config.txt", "one-hot,3,1.0\nmulti-hot,3,10,5,50,0.9\n")
    # features 0 and 2 share a table shape, 1 differs; 3 and 4 share shape but differ in dtype
    write(f"{m}/table_config.txt", "1024,16\n1024,32\n1024,16\n4096,8\n4096,8,half\n4096,8\n")
    write(f"{m}/schedule_config.txt", "\n".join(f"S{i}" for i in range(6)) + "\n")
    write(f"{m}/data/batch_sizes.txt", "2\n")
    for i in range(6):
        write(f"{m}/data/f{i}.txt", f"{i}\n{i},{i}\n")
    return m


def test_compress_clusters_by_config_line_shape_and_dtype(tmp_path):
    m = make_model(tmp_path)
    out = str(tmp_path / "small")
    run(os.path.join(EX, "compress.py"), "-m", m, "-o", out)
    assert open(f"{out}/feat_map.txt").read().split() == ["0,2", "1", "3,5", "4"]
    assert open(f"{out}/table_config.txt").read().split() == ["1024,16", "1024,32", "4096,8", "4096,8,half"]
    assert open(f"{out}/schedule_config.txt").read().split() == ["S0", "S1", "S3", "S4"]
    assert open(f"{out}/data_config.txt").read().split() == [
        "one-hot,1,1.0", "one-hot,1,1.0", "multi-hot,1,10,5,50,0.9", "multi-hot,1,10,5,50,0.9"]
    assert open(f"{out}/data/batch_sizes.txt").read() == "2\n"
    for new, old in enumerate([0, 1, 3, 4]):
        assert open(f"{out}/data/f{new}.txt").read() == open(f"{m}/data/f{old}.txt").read()


def test_decompress_spreads_results(tmp_path):
    m = make_model(tmp_path)
    small = str(tmp_path / "small")
    run(os.path.join(EX, "compress.py"), "-m", m, "-o", small)
    for k in range(4):
        write(f"{small}/output/f{k}/o2/result.txt", f"{k}.0 {k}.5")
        write(f"{small}/output/naive/f{k}/result.txt", f"n{k}")
    run(os.path.join(EX, "decompress.py"), "-i", small, "-o", m)
    want = {0: 0, 2: 0, 1: 1, 3: 2, 5: 2, 4: 3}
    for feat, rep in want.items():
        assert open(f"{m}/output/f{feat}/o2/result.txt").read() == f"{rep}.0 {rep}.5"
    assert not os.path.exists(f"{m}/output/naive")
    run(os.path.join(EX, "decompress.py"), "-i", small, "-o", m, "--naive")
    for feat, rep in want.items():
        assert open(f"{m}/output/naive/f{feat}/result.txt").read() == f"n{rep}"


def test_schedule_config_gen(tmp_path):
    m = make_model(tmp_path)
    out = str(tmp_path / "sched.txt")
    run(os.path.join(EX, "schedule_config_gen.py"), "-c", f"{m}/data_config.txt", "-s", out)
    lines = open(out).read().split()
    assert lines[:3] == ["OneHotSchedule"] * 3
    assert lines[3:] == ["ReduceByKeySchedule,OneBlockMultiSampleSchedule,WarpPerSampleSchedule"] * 3
    run(os.path.join(EX, "schedule_config_gen.py"), "-c", f"{m}/data_config.txt", "-s", out, "--names", "gfx950")
    from recflex_amd.schedules import SCHEDULE_MAPPING
    from recflex_amd.parser import parse_schedule_types
    types = parse_schedule_types(out, SCHEDULE_MAPPING)
    assert len(types) == 6 and all(len(t) >= 2 for t in types)


def test_table_config_generate(tmp_path):
    m = make_model(tmp_path)
    out = str(tmp_path / "tables.txt")
    script = os.path.join(ROOT, "data_synthesis", "table_config_generate.py")
    write(f"{m}/dc.txt", "one-hot,40,1.0\nmulti-hot,30,10,5,50,0.9\nmulti-hot-one-side,20,5,2,0.5\nmulti-hot-static,10,4,1.0\n")
    run(script, "-c", f"{m}/dc.txt", "-t", out, "--seed", "3")
    rows = [tuple(map(int, l.split(","))) for l in open(out).read().split()]
    assert [r for r, _ in rows] == [1024] * 40 + [4096] * 30 + [16384] * 20 + [4096] * 10
    assert all(d in (4, 8, 16, 32, 64, 128) for _, d in rows)
    first = open(out).read()
    run(script, "-c", f"{m}/dc.txt", "-t", out, "--seed", "3")
    assert open(out).read() == first                       # reproducible with a seed
    run(script, "-c", f"{m}/dc.txt", "-t", out, "-d", "64", "--dtype", "int8")
    assert set(open(out).read().split()) == {"1024,64,int8", "4096,64,int8", "16384,64,int8"}
    from recflex_amd.parser import parse_table_shapes, parse_table_dtypes
    assert len(parse_table_shapes(out)) == 100 and set(parse_table_dtypes(out)) == {"int8"}
