"""FR-Spec id lists on the host (no GPU): the file format and its rejections
(src/frspec.rs:101-117), the default location (src/frspec.rs:153-158) and the superset merge
of tools/merge_frspec.py:176-204, against a plain-Python statement of the same arithmetic."""
import collections
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _write_raw(path, ids, n=None):
    with open(path, "wb") as f:
        f.write(struct.pack("<I", len(ids) if n is None else n))
        f.write(np.asarray(ids, "<u4").tobytes())


def test_default_path_follows_the_environment(orn, monkeypatch):
    monkeypatch.delenv("ORNITH_FRSPEC", raising=False)
    monkeypatch.delenv("ORNITH_REFS", raising=False)
    assert orn.frspec_default_path() == "refs/frspec/ids_64k.bin"
    monkeypatch.setenv("ORNITH_REFS", "/data/refs")
    assert orn.frspec_default_path() == "/data/refs/frspec/ids_64k.bin"
    monkeypatch.setenv("ORNITH_FRSPEC", "/tmp/mine.bin")
    assert orn.frspec_default_path() == "/tmp/mine.bin"


def test_read_write_round_trip_and_rejections(orn, tmp_path):
    p = str(tmp_path / "ids.bin")
    assert orn.frspec_write_ids(p, [7, 3, 3, 900, 0], vocab=1000) == 4
    assert list(orn.frspec_read_ids(p)) == [0, 3, 7, 900]                # sorted, de-duplicated
    assert open(p, "rb").read() == struct.pack("<5I", 4, 0, 3, 7, 900)
    for ids, vocab, msg in (([], 10, "no ids"), (list(range(10)), 10, "not a pruning"), ([3, 10], 10, "outside")):
        with pytest.raises(orn.OrnithError, match=msg):
            orn.frspec_write_ids(p, ids, vocab)
    _write_raw(p, [1, 2, 3], n=5)
    with pytest.raises(orn.OrnithError, match="says 5 ids"):
        orn.frspec_read_ids(p)
    open(p, "wb").write(b"\x01\x00")
    with pytest.raises(orn.OrnithError, match="too short"):
        orn.frspec_read_ids(p)
    with pytest.raises(orn.OrnithError, match="cannot open"):
        orn.frspec_read_ids(str(tmp_path / "missing.bin"))


def test_merge_is_a_superset_with_the_reference_arithmetic(orn):
    rng = np.random.default_rng(0)
    vocab = 5000
    base = rng.permutation(vocab)[:1200].astype(np.uint32)
    # a corpus with a heavy head inside the list and a tail outside it, hapaxes included
    corpus = np.concatenate([rng.choice(base, 4000), rng.integers(0, vocab, 3000).astype(np.uint32)])
    extra = rng.permutation(vocab)[:300].astype(np.uint32)
    for min_count in (1, 2, 3):
        merged, st = orn.frspec_merge(base, corpus, min_count, extra, vocab)
        inside = set(int(i) for i in base)
        seen = collections.Counter(int(i) for i in corpus)
        missing = {i: v for i, v in seen.items() if i not in inside}
        keep = sorted(i for i, v in missing.items() if v >= min_count)
        want = sorted(inside | set(keep) | set(int(i) for i in extra))
        assert list(merged) == want
        assert set(int(i) for i in base) <= set(int(i) for i in merged)          # it only adds
        assert st.n_merged == len(want) and st.corpus_tokens == len(corpus)
        assert st.covered_before == sum(v for i, v in seen.items() if i in inside)
        assert st.covered_after == st.covered_before + sum(missing[i] for i in keep)
        assert st.missing_distinct == len(missing) and st.missing_kept == len(keep)
        assert st.extra_new == len(set(int(i) for i in extra) - inside)
    merged, st = orn.frspec_merge(base, None, 2, extra, vocab)                    # script only
    assert list(merged) == sorted(set(int(i) for i in base) | set(int(i) for i in extra)) and st.corpus_tokens == 0
    with pytest.raises(orn.OrnithError, match="nothing to add"):
        orn.frspec_merge(base, None, 2, None, vocab)
    with pytest.raises(orn.OrnithError, match="outside"):
        orn.frspec_merge(base, np.array([vocab], np.uint32), 1, None, vocab)
    with pytest.raises(orn.OrnithError, match="not a pruning"):
        orn.frspec_merge(base, np.arange(vocab, dtype=np.uint32), 1, None, vocab)


def test_merge_tool_writes_the_merged_list(orn, tmp_path):
    vocab = 1000
    base, corp, out = str(tmp_path / "base.bin"), str(tmp_path / "c.u32"), str(tmp_path / "plus.bin")
    orn.frspec_write_ids(base, list(range(0, 200)), vocab)
    np.array([5, 5, 300, 300, 301, 999, 999, 999], "<u4").tofile(corp)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "ornith-rs_amd", "merge_frspec.py"), "--base", base, "--vocab",
                        str(vocab), "--out", out, corp], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert list(orn.frspec_read_ids(out)) == list(range(200)) + [300, 999]
    assert "coverage with the merged list: 87.5%" in r.stdout
