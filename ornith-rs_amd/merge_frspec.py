"""Extend an FR-Spec draft vocabulary with what a corpus needs and the list lacks.

    python ornith-rs_amd/merge_frspec.py --base ids_64k.bin --vocab 248320 \
        [--min-count 2] [--extra more_ids.bin] [--out ids_64k_plus.bin] corpus_a.u32 corpus_b.npy ...

The counterpart of the reference's tools/merge_frspec.py (lines 74-92, 176-204) on TOKEN IDS:
a corpus here is a file of token ids (raw little-endian u32, or a .npy integer array) --
tokenizing text is the caller's business. The merged list only ever adds to the base list
(every id the corpus used at least --min-count times and the base lacks, plus --extra, an id
list file such as every id of one script), so what the base covered stays covered by
construction; it is written sorted and de-duplicated in the same `u32 n, n x u32` format and
must remain a strict pruning of the vocabulary. The arithmetic runs in the library
(ornith_frspec_merge / ornith_frspec_write_ids).
"""
import argparse
import importlib
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def read_corpus(path):
    if path.endswith(".npy"):
        a = np.load(path, allow_pickle=False)
        if not np.issubdtype(a.dtype, np.integer):
            sys.exit(f"{path}: not an integer array")
        return a.astype(np.uint32).reshape(-1)
    return np.fromfile(path, dtype="<u4")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("corpus", nargs="*", help="files of token ids (raw u32 or .npy)")
    ap.add_argument("--base", default=None, help="the list to extend (default: the library's default path)")
    ap.add_argument("--extra", default=None, help="an id list file whose ids are all added")
    ap.add_argument("--vocab", type=int, default=248320)
    ap.add_argument("--min-count", type=int, default=2)
    ap.add_argument("--out", default=None, help="default: <base>_plus.bin")
    a = ap.parse_args()
    orn = importlib.import_module("ornith-rs_amd")
    base_path = a.base or orn.frspec_default_path()
    out = a.out or os.path.splitext(base_path)[0] + "_plus.bin"
    if not a.corpus and not a.extra:
        sys.exit("nothing to add: give a corpus, or --extra, or both")
    base = orn.frspec_read_ids(base_path)
    corpus = np.concatenate([read_corpus(p) for p in a.corpus]) if a.corpus else None
    extra = orn.frspec_read_ids(a.extra) if a.extra else None
    merged, st = orn.frspec_merge(base, corpus, a.min_count, extra, a.vocab)
    n = orn.frspec_write_ids(out, merged, a.vocab)
    if st.corpus_tokens:
        print(f"corpus: {len(a.corpus)} files, {st.corpus_tokens} tokens")
        print(f"  coverage with {base_path}: {100 * st.covered_before / st.corpus_tokens:.1f}%")
        print(f"  missing ids: {st.missing_distinct} distinct, {st.missing_kept} of them seen >= {a.min_count}")
        print(f"  coverage with the merged list: {100 * st.covered_after / st.corpus_tokens:.1f}%")
    if extra is not None:
        print(f"  --extra {a.extra}: {st.extra_new} ids not already in the list")
    print(f"{out}: {n} ids ({n / a.vocab:.4f} of the vocabulary, +{100 * (n - len(base)) / len(base):.1f}%)")


if __name__ == "__main__":
    main()
