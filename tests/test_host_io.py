"""The command line's host I/O layer (csrc/io_utils.cpp) on the CPU: the TSV readers' id mapping and test-set rules
(io_utils.h:81-111,183-238) and the two model-file layouts (io_utils.h:242-332), whose numbers must read exactly as
`ostream << float` writes them (%g)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "icdm-2021_mascot_amd", "csrc")


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("host_io") / "host_io_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-pthread", "-o", exe, os.path.join(ROOT, "tests", "host_io_check.cpp"),
                    os.path.join(CSRC, "io_utils.cpp")], check=True)
    return exe


def c_format(v):
    """'%g' of a binary32 value, as printf and the stream's default float formatting give it."""
    return "%g" % float(v)


@pytest.mark.parametrize("k", [4, 64])
def test_readers_and_model_files(driver, tmp_path, k):
    train = tmp_path / "train.tsv"
    test = tmp_path / "test.tsv"
    # users 40, 7, 1000 and items 5, 900, 3 in first-seen order; item 2 and user 8 never occur in training
    train_lines = [(40, 5, 3.0), (7, 900, 4.5), (40, 900, 1.0), (1000, 3, 5.0), (7, 5, 2.0), (1000, 900, 0.5)]
    train.write_text("".join("%d\t%d\t%g\n" % t for t in train_lines))
    # an unseen user, an unseen item, a duplicate (the later line wins), and lines out of (user, item) order
    test_lines = [(1000, 900, 2.0), (8, 5, 1.0), (40, 2, 1.0), (7, 3, 3.5), (40, 3, 4.0), (7, 3, 2.5), (40, 5, 1.5)]
    test.write_text("".join("%d\t%d\t%g\n" % t for t in test_lines))
    out = str(tmp_path / "model")
    r = subprocess.run([driver, str(train), str(test), out, str(k)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = r.stdout.splitlines()
    summary = [l for l in lines if l.startswith("users ")][0].split()
    assert summary[1] == "3" and summary[3] == "3" and summary[5] == "6"
    users = {int(l.split()[1]): int(l.split()[3]) for l in lines if l.startswith("user ")}
    items = {int(l.split()[1]): int(l.split()[3]) for l in lines if l.startswith("item ")}
    assert users == {0: 40, 1: 7, 2: 1000} and items == {0: 5, 1: 900, 2: 3}              # first-seen order
    got_train = [tuple(l.split()[1:]) for l in lines if l.startswith("train ")]
    u2d, i2d = {v: key for key, v in users.items()}, {v: key for key, v in items.items()}
    assert got_train == [(str(u2d[u]), str(i2d[i]), "%.9g" % r_) for u, i, r_ in train_lines]
    # test set: unseen ids dropped (and listed), duplicates folded, ordered by dense user then dense item
    got_test = [(int(a), int(b), float(c)) for a, b, c in (l.split()[1:] for l in lines if l.startswith("test "))]
    want = {}
    for u, i, r_ in test_lines:
        if u in u2d and i in i2d:
            want[(u2d[u], i2d[i])] = r_
    assert got_test == [(u, i, want[(u, i)]) for u, i in sorted(want)]
    assert (tmp_path / "remove_user.txt").read_text().split() == ["8"]
    assert (tmp_path / "remove_item.txt").read_text().split() == ["2"]
    # the values the driver put into P and Q
    vals = np.fromfile(out + ".values", np.float32)
    P, Q = vals[:3 * k].reshape(3, k), vals[3 * k:].reshape(3, k)
    # <out>_reconst.txt: header, then the rows in dense order
    text = open(out + "_reconst.txt").read()
    head, body_p, body_q = text.split("\n")
    assert head == "3 3 %d" % k
    assert body_p == "".join(c_format(v) + " " for v in P.reshape(-1))
    assert body_q == "".join(c_format(v) + " " for v in Q.reshape(-1))
    # <out>.txt: rows by original id, zeros for ids that never occurred
    text = open(out + ".txt").read()
    head, body_p, body_q = text.split("\n")
    assert head == "1001 901 %d" % k
    tok = body_p.split(" ")
    assert tok[-1] == "" and len(tok) == 1001 * k + 1
    for orig in range(1001):
        row = tok[orig * k:(orig + 1) * k]
        assert row == ([c_format(v) for v in P[u2d[orig]]] if orig in u2d else ["0"] * k), orig
    tok = body_q.split(" ")
    assert len(tok) == 901 * k + 1
    for orig in (0, 2, 3, 4, 5, 6, 899, 900):
        row = tok[orig * k:(orig + 1) * k]
        assert row == ([c_format(v) for v in Q[i2d[orig]]] if orig in i2d else ["0"] * k), orig
    # reconst_<testfile>: the kept test ratings in the dense index space, user first
    rec = (tmp_path / "reconst_test.tsv").read_text().splitlines()
    assert rec == ["%d\t%d\t%s" % (u, i, c_format(np.float32(want[(u, i)]))) for u, i in sorted(want)]
    assert [l for l in lines if l.startswith("reread ")][0] == "reread users 3 items 3 k %d p %d q %d" % (k, 3 * k, 3 * k)


def _dump(driver, train, test, out):
    r = subprocess.run([driver, str(train), str(test), out, "4"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = r.stdout.splitlines()
    users = {int(l.split()[1]): int(l.split()[3]) for l in lines if l.startswith("user ")}
    items = {int(l.split()[1]): int(l.split()[3]) for l in lines if l.startswith("item ")}
    # ratings are printed with nine significant digits, which identify a binary32 value
    got_train = [(int(a), int(b), float(np.float32(c))) for a, b, c in (l.split()[1:] for l in lines if l.startswith("train "))]
    got_test = [(int(a), int(b), float(np.float32(c))) for a, b, c in (l.split()[1:] for l in lines if l.startswith("test "))]
    summary = [l for l in lines if l.startswith("users ")][0].split()
    return users, items, got_train, got_test, dict(zip(summary[0::2], summary[1::2]))


@pytest.mark.parametrize("dirname", ["netflix_prize", "ml-25M", "plain"])
def test_item_first_column_order_by_path(driver, tmp_path, dirname):
    """io_utils.h:40-47: a path that contains "netflix" or "25M" holds the item in the first column and the user in the
    second; any other path user first.  The same lines therefore load transposed."""
    d = tmp_path / dirname
    d.mkdir()
    train, test = d / "train.tsv", d / "test.tsv"
    lines = [(11, 500, 4.0), (12, 500, 3.0), (11, 600, 1.5), (13, 700, 5.0)]
    train.write_text("".join("%d\t%d\t%g\n" % t for t in lines))
    test.write_text("11\t700\t2.5\n13\t500\t1.0\n99\t500\t3.0\n")
    users, items, got_train, got_test, summary = _dump(driver, train, test, str(tmp_path / ("m_" + dirname)))
    swapped = dirname != "plain"
    first, second = [a for a, _, _ in lines], [b for _, b, _ in lines]
    want_users = list(dict.fromkeys(second if swapped else first))          # first-seen order of the user column
    want_items = list(dict.fromkeys(first if swapped else second))
    assert [users[i] for i in range(len(users))] == want_users
    assert [items[i] for i in range(len(items))] == want_items
    u2d, i2d = {v: i for i, v in enumerate(want_users)}, {v: i for i, v in enumerate(want_items)}
    assert got_train == [((u2d[b], i2d[a], r) if swapped else (u2d[a], i2d[b], r)) for a, b, r in lines]
    if swapped:      # test lines are (item, user, rating): item 11 user 700, item 13 user 500; item 99 never occurred
        assert got_test == sorted([(u2d[700], i2d[11], 2.5), (u2d[500], i2d[13], 1.0)])
        assert (d / "remove_item.txt").read_text().split() == ["99"] and (d / "remove_user.txt").read_text().split() == []
    else:
        assert got_test == sorted([(u2d[11], i2d[700], 2.5), (u2d[13], i2d[500], 1.0)])
        assert (d / "remove_user.txt").read_text().split() == ["99"]
    assert summary["missing"] == "1"


def test_yahoo_block_format(driver, tmp_path):
    """io_utils.h:49-79,139-181: a path that contains "Yahoo" holds blocks "user|count" followed by count lines
    "item<TAB>rating" with ratings 0..100, which are mapped to rating / 25 + 1; ids are numbered in first-seen order;
    in the test file a rating of an unknown item is dropped and counted, a block of an unknown user is counted whole."""
    d = tmp_path / "YahooMusic"
    d.mkdir()
    train, test = d / "train.txt", d / "test.txt"
    train.write_text("7|3\n100\t90\n200\t0\n300\t50\n5|1\n200\t100\n9|2\n300\t25\n400\t75\n")
    test.write_text("5|2\n100\t80\n999\t10\n8|2\n100\t1\n200\t2\n9|1\n100\t30\n")
    users, items, got_train, got_test, summary = _dump(driver, train, test, str(tmp_path / "m"))
    assert [users[i] for i in range(3)] == [7, 5, 9] and [items[i] for i in range(4)] == [100, 200, 300, 400]
    f = lambda r: float(np.float32(np.float32(r) / np.float32(25.0)) + np.float32(1.0))
    assert got_train == [(0, 0, f(90)), (0, 1, f(0)), (0, 2, f(50)), (1, 1, f(100)), (2, 2, f(25)), (2, 3, f(75))]
    assert f(0) == 1.0 and f(100) == 5.0 and f(90) == 4.599999904632568
    # user 5: item 100 kept, item 999 unknown (1 missing); user 8 unknown: its 2 ratings missing, and the block after it parses
    assert got_test == [(1, 0, f(80)), (2, 0, f(30))]
    assert summary["missing"] == "3" and summary["test"] == "2"


def test_many_rows_are_written_in_order(driver, tmp_path):
    """More rows than one formatting block per thread: the blocks must land in the file in row order."""
    n_users, n_items, k = 70_001, 3, 2
    train = tmp_path / "train.tsv"
    train.write_text("".join("%d\t%d\t1\n" % (u, u % n_items) for u in range(n_users)))
    test = tmp_path / "test.tsv"
    test.write_text("0\t0\t1\n")
    out = str(tmp_path / "m")
    r = subprocess.run([driver, str(train), str(test), out, str(k)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    vals = np.fromfile(out + ".values", np.float32)
    P = vals[:n_users * k]
    head, body_p, body_q = open(out + "_reconst.txt").read().split("\n")
    assert head == "%d %d %d" % (n_users, n_items, k)
    assert body_p == "".join(c_format(v) + " " for v in P)


def test_round_half_away_identity_is_exhaustive(tmp_path):
    """The fixed-point kernels round with trunc(x + copysign(pred(0.5), x)); the reference calls roundf.  All 2^32 bit
    patterns agree."""
    exe = str(tmp_path / "round_identity_check")
    subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe, os.path.join(ROOT, "tests", "round_identity_check.c"), "-lm"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and r.stdout.strip() == "0", r.stdout + r.stderr


def test_scale_index_from_bits_equals_its_definition(tmp_path):
    """The MuPPET kernels take floor(log2(bound / x)) from the exponent and mantissa of x; the reference divides and calls
    log2f (muppet/muppet_sgd_kernel.h:7-18).  Outside 64 ulps around the threshold mantissa (where the kernels evaluate the
    definition) the two agree for every exponent, both signs, zeros, subnormals, infinities and NaN, at every bit width."""
    exe = str(tmp_path / "scale_index_identity_check")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-o", exe, os.path.join(ROOT, "tests", "scale_index_identity_check.c"), "-lm"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and r.stdout.strip() == "0", r.stdout + r.stderr


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits without touching a device."""
    import subprocess
    import sys
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout == ""
