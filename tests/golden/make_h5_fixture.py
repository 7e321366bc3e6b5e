"""Writes tests/golden/h5py_layout.hdf5.gz and h5py_layout_expected.npz with the real h5py.

Run once, in the build container, with the interpreter that has h5py (3.3.0 over libhdf5 1.10):

    /opt/conda/bin/python3.9 tests/golden/make_h5_fixture.py

The file is laid out by the calls the reference's dataset manager makes
(classes/data_manager.py:287-312: one group `convo_{id}` per conversation, attributes
`content_sha` and `sample`, dataset `distributions` float16 gzip-6 and dataset `indices` uint32
gzip-6, both with h5py's automatic chunk shape; :147,153: file attributes `vocab_family` and
`topk`).  Besides two conversations of realistic shape it holds a dense-mode conversation without
`indices`, a conversation whose datasets were deleted and created again (the merge path, :303-311)
and enough small groups that the root group's B-tree has two levels.  The arrays are seeded (few distinct values, to keep the files small); the
.npz holds what a reader must return, bit for bit.
"""
import gzip
import os

import h5py
import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
rng = np.random.default_rng(20240611)
expected = {}


def save(f, cid, rows, width, with_idx=True, sha=None, sample=None):
    g = f.require_group(f"convo_{cid}")
    if sha is not None:
        g.attrs["content_sha"] = sha
    if sample is not None:
        g.attrs["sample"] = sample
    # few distinct values, so that the fixture stays small; rows differ from each other
    d = (-(rng.integers(0, 12, size=(rows, width)) + np.arange(rows)[:, None] % 7) / 4).astype(np.float16)
    if "distributions" in g:
        del g["distributions"]
    g.create_dataset("distributions", data=d, compression="gzip", compression_opts=6, dtype=np.float16)
    expected[f"d{cid}"] = d
    if with_idx:
        i = (rng.integers(0, 9, size=(rows, width)) * 16896 + np.arange(width)[None, :]).astype(np.uint32)
        if "indices" in g:
            del g["indices"]
        g.create_dataset("indices", data=i, compression="gzip", compression_opts=6, dtype=np.uint32)
        expected[f"i{cid}"] = i


path = os.path.join(HERE, "h5py_layout.hdf5")
with h5py.File(path, "w") as f:
    f.attrs["vocab_family"] = "llama_3"
    f.attrs["topk"] = 200
    save(f, 0, 37, 8, sha="3f2a" * 16, sample="system: hi\nuser: é中")
    save(f, 3, 160, 200, sha="00ff" * 16, sample="")
    save(f, 12, 5, 4096, with_idx=False, sha="abcd" * 16, sample="dense")
    save(f, 7, 19, 8, sha="1234" * 16, sample="first")
    save(f, 7, 23, 8)                      # replaced by a merge: new datasets, attributes kept
    for cid in range(1000, 1300):          # > 256 groups: two B-tree levels under the root
        g = f.create_group(f"convo_{cid}")
        g.attrs["content_sha"] = f"{cid:064x}"
    save(f, 1299, 3, 8)
    for cid in (1005, 1150):               # removed conversations (clear_ids)
        del f[f"convo_{cid}"]
expected["removed"] = np.array([1005, 1150])
with open(path, "rb") as src, gzip.GzipFile(path + ".gz", "wb", mtime=0) as dst:
    dst.write(src.read())
print("hdf5 bytes", os.path.getsize(path), "gz bytes", os.path.getsize(path + ".gz"))
os.remove(path)
np.savez_compressed(os.path.join(HERE, "h5py_layout_expected.npz"), **expected)
