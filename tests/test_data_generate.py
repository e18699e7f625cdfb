"""CPU test of ``data_synthesis/data_generate.py``: the writer of the dataset text format
(reference: ``data_synthesis/data_generate.py:42-80,120-178``, ``data_synthesis/README.md:7-14``).
Each of the four ``data_config`` feature types produces files that the parser reads back --
``batch_sizes.txt`` sums to the line count of every ``f{i}.txt``, an empty line is an absent
sample -- with the pooling factors, coverage and index range the config asks for; a seed
reproduces the files and existing files are kept."""

import os
import subprocess
import sys

import numpy as np
import pytest

from helpers import ROOT
from recflex_amd.host import RecomHost
from recflex_amd.parser import parse_raw_data_batches
from recflex_amd.utils import get_data_fnames

SCRIPT = os.path.join(ROOT, "data_synthesis", "data_generate.py")

# type, count, params  (README.md:7-14 of the reference's data_synthesis)
DATA_CONFIG = ("one-hot,2,0.8\n"
               "multi-hot,2,20,10,60,0.9\n"
               "multi-hot-static,1,7,0.5\n"
               "multi-hot-one-side,1,5,4,1.0\n")
TABLE_CONFIG = "500,8\n500,8\n3000,16\n3000,16\n64,4\n900,32\n"
ROWS = [500, 500, 3000, 3000, 64, 900]
QUERIES, QUERY_MAX = 40, 96


def generate(out_dir, tmp_path, seed=1000):
    cfg, tab = tmp_path / "data_config.txt", tmp_path / "table_config.txt"
    cfg.write_text(DATA_CONFIG)
    tab.write_text(TABLE_CONFIG)
    subprocess.run([sys.executable, SCRIPT, "-c", str(cfg), "-t", str(tab), "-o", str(out_dir),
                    "-s", str(seed), "--num_queries", str(QUERIES), "--query_mean", "48",
                    "--query_stddev", "2", "--query_max", str(QUERY_MAX)],
                   check=True, cwd=ROOT, stdout=subprocess.DEVNULL)
    return str(out_dir)


def read_bags(data_dir):
    """Per feature: list of bag lengths and the flat indices, through the text front end."""
    sizes = [int(l) for l in open(f"{data_dir}/batch_sizes.txt") if l.strip()]
    host = RecomHost()
    feats = []
    for fname in get_data_fnames(data_dir):
        lines = open(fname).read().split("\n")
        assert lines[-1] == "" and len(lines) - 1 == sum(sizes), fname     # one line per sample
        idx, off = host.parse_lines(lines[:-1])
        lens = np.diff(off)
        assert [len(l) == 0 for l in lines[:-1]] == (lens == 0).tolist()    # empty line <=> empty bag
        feats.append((lens, idx))
    return sizes, feats


def test_every_feature_type_is_written_and_read_back(tmp_path):
    d = generate(tmp_path / "data", tmp_path)
    sizes, feats = read_bags(d)
    assert len(sizes) == QUERIES and all(1 <= s <= QUERY_MAX for s in sizes)
    assert len(feats) == 6
    total = sum(sizes)
    for (lens, idx), rows in zip(feats, ROWS):
        assert len(lens) == total and idx.min() >= 0 and idx.max() < rows

    def coverage_ok(lens, coverage):
        present = int((lens > 0).sum())
        sigma = np.sqrt(total * coverage * (1 - coverage))
        return abs(present - total * coverage) <= 3 * sigma + 1

    # one-hot: exactly one index where present
    for lens, _ in feats[0:2]:
        assert set(np.unique(lens)) <= {0, 1} and coverage_ok(lens, 0.8)
    # multi-hot: pooling factor from N(20, 10) cut to [0, 60]; a drawn factor of 0 also gives an
    # empty line, so the share of non-empty bags is a little under the coverage
    for lens, _ in feats[2:4]:
        assert lens.max() <= 60 and 14 < lens[lens > 0].mean() < 26
        assert (lens > 0).mean() <= 0.9 + 3 * np.sqrt(0.09 / total) and (lens > 0).mean() > 0.8
    # multi-hot-static: exactly 7 where present
    lens, _ = feats[4]
    assert set(np.unique(lens)) <= {0, 7} and coverage_ok(lens, 0.5)
    # multi-hot-one-side: N(5, 4) cut at 0, every sample present
    lens, _ = feats[5]
    assert lens.min() >= 0 and 3.5 < lens.mean() < 7.5 and lens.max() < 5 + 6 * 4
    # the features of one group share pooling factors and absent samples, not the indices
    assert (feats[0][0] == feats[1][0]).all() and (feats[2][0] == feats[3][0]).all()
    assert not np.array_equal(feats[2][1], feats[3][1])
    # popular rows: a power-law probability vector, not uniform -- the most frequent row of the
    # 64-row table is drawn clearly more often than 1 / 64 of the time
    counts = np.bincount(feats[4][1], minlength=64)
    assert counts.max() > 1.5 * counts.sum() / 64

    # the reader used by tune.py / test.py sees the same batches
    raw = parse_raw_data_batches(f"{d}/batch_sizes.txt", get_data_fnames(d), QUERIES, seed=0,
                                 feat_major=True)
    assert len(raw) == 6 and [len(b) for b in raw[0]] == sizes


def test_seed_reproduces_the_files_and_existing_files_are_kept(tmp_path):
    a = generate(tmp_path / "a", tmp_path)
    b = generate(tmp_path / "b", tmp_path)
    c = generate(tmp_path / "c", tmp_path, seed=77)
    names = ["batch_sizes.txt"] + [f"f{i}.txt" for i in range(6)]
    for n in names:
        assert open(f"{a}/{n}").read() == open(f"{b}/{n}").read(), n
    assert any(open(f"{a}/{n}").read() != open(f"{c}/{n}").read() for n in names)
    # resume: a second run leaves what is there alone and writes only what is missing
    with open(f"{a}/f0.txt", "w") as f:
        f.write("kept\n")
    os.remove(f"{a}/f3.txt")
    generate(tmp_path / "a", tmp_path)
    assert open(f"{a}/f0.txt").read() == "kept\n"
    assert open(f"{a}/f3.txt").read() == open(f"{b}/f3.txt").read()
    assert not [n for n in os.listdir(a) if n.endswith(".tmp")]


def test_config_and_table_list_must_describe_the_same_features(tmp_path):
    cfg, tab = tmp_path / "data_config.txt", tmp_path / "table_config.txt"
    cfg.write_text("one-hot,2,1.0\n")
    tab.write_text("10,4\n10,4\n10,4\n")
    proc = subprocess.run([sys.executable, SCRIPT, "-c", str(cfg), "-t", str(tab), "-o", str(tmp_path / "o"),
                           "--num_queries", "2"], cwd=ROOT, capture_output=True, text=True)
    assert proc.returncode != 0 and "describes 2 features" in proc.stderr
    cfg.write_text("no-such-type,3,1.0\n")
    proc = subprocess.run([sys.executable, SCRIPT, "-c", str(cfg), "-t", str(tab), "-o", str(tmp_path / "p"),
                           "--num_queries", "2"], cwd=ROOT, capture_output=True, text=True)
    assert proc.returncode != 0 and "unknown feature type" in proc.stderr
