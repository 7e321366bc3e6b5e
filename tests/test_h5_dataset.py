"""The dataset file format (`distributions.hdf5`, classes/data_manager.py:287-353) read and written
without h5py.  Pinned three ways: a file written by the real h5py 3.3 / libhdf5 1.10 with the
reference's calls (tests/golden/make_h5_fixture.py) must decode bit for bit; files written here must
round-trip; and, where an interpreter with h5py is installed (the build container), the real
library must read what is written here, append to it, and have its own files appended to."""
import gzip
import os
import subprocess

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

import llm_distillery_amd as D
from llm_distillery_amd import h5_format as F
from llm_distillery_amd.h5_dataset import DistributionStore

GOLD = os.path.join(os.path.dirname(__file__), "golden")
H5PY_PYTHON = "/opt/conda/bin/python3.9"


def _h5py_available():
    if not os.path.exists(H5PY_PYTHON):
        return False
    try:
        return subprocess.run([H5PY_PYTHON, "-c", "import h5py"], capture_output=True, timeout=60).returncode == 0
    except (OSError, subprocess.TimeoutExpired):
        return False


needs_h5py = pytest.mark.skipif(not _h5py_available(), reason="no interpreter with h5py on this machine")


def _run_h5py(code, *args):
    r = subprocess.run([H5PY_PYTHON, "-c", code, *args], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout


@pytest.fixture()
def fixture_file(tmp_path):
    path = tmp_path / "distributions.hdf5"
    path.write_bytes(gzip.open(os.path.join(GOLD, "h5py_layout.hdf5.gz")).read())
    return str(path)


@pytest.fixture(scope="module")
def expected():
    return np.load(os.path.join(GOLD, "h5py_layout_expected.npz"))


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16 if a.dtype.itemsize == 2 else np.uint32)


def _convos(seed, ids, K=16, max_rows=50):
    rng = np.random.default_rng(seed)
    out = {}
    for cid in ids:
        n = int(rng.integers(0, max_rows))
        out[cid] = ((rng.standard_normal((n, K)) * 3 - 5).astype(np.float16), rng.integers(0, 152064, (n, K)).astype(np.uint32))
    return out


# ---------------------------------------------------------------------------------------------
# the reader against a file made by h5py
# ---------------------------------------------------------------------------------------------
def test_reads_h5py_file_bit_exact(fixture_file, expected):
    with DistributionStore(fixture_file, "r") as s:
        ids = s.get_available_ids()
        assert len(ids) == 302 and set(expected["removed"]).isdisjoint(ids)     # two B-tree levels under the root
        assert {0, 3, 7, 12, 1000, 1299} <= set(ids)
        assert s.get_vocab_family() == "llama_3" and s.get_topk() == 200 and s.get_dataset_attr("nothing") is None
        assert s.has_data()
        for cid in (0, 3, 7, 12, 1299):
            d, i = s.load_id(cid, storage=True)
            assert d.dtype == np.float16 and np.array_equal(_bits(d), _bits(expected[f"d{cid}"]))
            if f"i{cid}" in expected.files:
                assert i.dtype == np.uint32 and np.array_equal(i, expected[f"i{cid}"])
            else:
                assert i is None                                                  # dense-mode conversation
            d32, i64 = s.load_id(cid)                                             # the reference's casts (:323-324)
            assert d32.dtype == np.float32 and np.array_equal(d32, expected[f"d{cid}"].astype(np.float32))
            assert i is None or (i64.dtype == np.int64 and np.array_equal(i64, expected[f"i{cid}"]))
        assert s.shape_of(3) == ((160, 200), True) and s.shape_of(12) == ((5, 4096), False)
        assert s.group_attrs(0) == {"content_sha": "3f2a" * 16, "sample": "system: hi\nuser: é中"}
        assert s.group_attrs(7) == {"content_sha": "1234" * 16, "sample": "first"}   # kept across the merge rewrite
        shas = s.get_available_shas()
        assert shas[1001] == f"{1001:064x}" and len(shas) == 302
        with pytest.raises(ValueError, match="not found"):
            s.load_id(1005)
        with pytest.raises(ValueError, match="no distributions"):
            s.load_id(1000)
        with pytest.raises(PermissionError):
            s.save_data(np.zeros((1, 8), np.float16), 5)


def test_outgoing_batch_matches_reference_layout(fixture_file, expected):
    with DistributionStore(fixture_file, "r") as s:
        padded, idx, pad = s.make_outgoing_batch([0, 7, 1299])
        assert padded.dtype == np.float32 and padded.shape == (3, 37, 8) and pad == [37, 23, 3]
        for b, cid in enumerate((0, 7, 1299)):
            assert np.array_equal(padded[b, :pad[b]], expected[f"d{cid}"].astype(np.float32))
            assert not padded[b, pad[b]:].any()                                   # zero padding (:341)
            assert idx[b].dtype == np.int64 and np.array_equal(idx[b], expected[f"i{cid}"])
        vals, ids, counts = s.packed_batch([0, 7, 1299], pin=False)
        assert counts == pad and vals.dtype.is_floating_point and vals.element_size() == 2 and ids.element_size() == 4
        assert np.array_equal(_bits(vals.numpy()), _bits(np.concatenate([expected[f"d{c}"] for c in (0, 7, 1299)])))
        assert np.array_equal(ids.numpy(), np.concatenate([expected[f"i{c}"] for c in (0, 7, 1299)]).astype(np.int32))
        # the packed tensors feed the same consumer as the reference's tuple
        t_ref = D.teachers_from_outgoing_batch(padded, idx, pad, "cpu")
        cuts = np.cumsum([0] + counts)
        for b in range(3):
            assert np.array_equal(_bits(t_ref[b][0].numpy()), _bits(vals[cuts[b]:cuts[b + 1]].numpy()))
            assert np.array_equal(t_ref[b][1].numpy(), ids[cuts[b]:cuts[b + 1]].numpy())
        with pytest.raises(ValueError, match="different top-K"):
            s.packed_batch([0, 3], pin=False)
        with pytest.raises(ValueError, match="dense-mode"):
            s.packed_batch([12], pin=False)


def test_prefetcher_yields_the_batches_in_order_and_ends(fixture_file, expected):
    from llm_distillery_amd import BatchPrefetcher
    batches = [[0], [7, 1299], [1299, 0, 7]]
    with DistributionStore(fixture_file, "r", workers=2) as s:
        with BatchPrefetcher(s, batches, "cpu", depth=1) as pf:
            got = list(pf)
            with pytest.raises(StopIteration):
                next(pf)
        assert len(got) == 3
        for ids, teachers in zip(batches, got):
            assert len(teachers) == len(ids)
            for cid, (v, i) in zip(ids, teachers):
                assert np.array_equal(_bits(v.numpy()), _bits(expected[f"d{cid}"])) and np.array_equal(i.numpy(), expected[f"i{cid}"].astype(np.int32))
        with BatchPrefetcher(s, batches[:2], "cpu", depth=2, loop=True) as pf:      # read-only mode: round and round
            seen = [len(next(pf)) for _ in range(7)]
        assert seen == [1, 2, 1, 2, 1, 2, 1]
        with BatchPrefetcher(s, [[0], [424242]], "cpu") as pf:                      # worker errors surface at the consumer
            next(pf)
            with pytest.raises(ValueError, match="not found"):
                next(pf)


# ---------------------------------------------------------------------------------------------
# the writer: round trips
# ---------------------------------------------------------------------------------------------
def test_roundtrip_many_groups_small_chunks_and_reopen(tmp_path):
    path = str(tmp_path / "d.hdf5")
    data = _convos(1, list(range(700)) + [10 ** 9])        # > 8 * 32 groups: two B-tree levels
    with DistributionStore(path, "w", chunk_bytes=256) as s:     # a few rows per chunk: chunk B-trees get several leaves
        s.set_vocab_family("mistral"); s.set_topk(16)
        for cid, (d, i) in data.items():
            s.save_data(d, cid, i, content_sha=f"{cid:x}", sample=f"s{cid}")
        big = (np.arange(300 * 16).reshape(300, 16) % 251 / 8).astype(np.float16)
        s.save_data(big, 5, np.arange(300 * 16, dtype=np.uint32).reshape(300, 16))      # 150 chunks: two chunk B-tree levels
        data[5] = (big, np.arange(300 * 16, dtype=np.uint32).reshape(300, 16))
        assert np.array_equal(_bits(s.load_id(3, storage=True)[0]), _bits(data[3][0]))  # readable before the flush
    with DistributionStore(path, "r") as s:
        assert sorted(s.get_available_ids()) == sorted(data) and s.get_topk() == 16 and s.get_vocab_family() == "mistral"
        for cid, (d, i) in data.items():
            dd, ii = s.load_id(cid, storage=True)
            assert dd.shape == d.shape and np.array_equal(_bits(dd), _bits(d)) and np.array_equal(ii, i)
        assert s.group_attrs(10 ** 9) == {"content_sha": f"{10 ** 9:x}", "sample": f"s{10 ** 9}"}


def test_append_merge_rename_clear(tmp_path):
    path = str(tmp_path / "d.hdf5")
    data = _convos(2, range(6), K=8)
    with DistributionStore(path, "a") as s:
        assert not s.has_data() and s.get_topk() is None
        s.set_vocab_family("llama_3"); s.set_topk(8)
        for cid, (d, i) in data.items():
            s.save_data(d, cid, i, content_sha=f"sha{cid}", sample="x")
    size0 = os.path.getsize(path)
    new = _convos(3, [2, 9], K=8)
    with DistributionStore(path, "a") as s:
        s.save_data(new[2][0], 2, new[2][1])                           # merge result replaces the datasets, attributes stay
        s.save_data(new[9][0], 9, new[9][1], content_sha="sha9", sample="")
        s.update_shas({0: "fresh", 77: "ignored"})                     # unknown ids are skipped (:277-281)
        s.rename_ids({0: 1, 1: 0, 5: 50})                              # a swap and a move at once (:370-376)
        with pytest.raises(ValueError, match="exists"):
            s.rename_ids({3: 4})
        with pytest.raises(KeyError):
            s.rename_ids({1234: 1})
    data[2] = new[2]; data[9] = new[9]
    data[0], data[1] = data[1], data[0]
    data[50] = data.pop(5)
    assert os.path.getsize(path) > size0
    with DistributionStore(path, "a") as s:
        assert sorted(s.get_available_ids()) == sorted(data)
        for cid, (d, i) in data.items():
            dd, ii = s.load_id(cid, storage=True)
            assert np.array_equal(_bits(dd), _bits(d)) and np.array_equal(ii, i)
        shas = s.get_available_shas()
        assert shas[1] == "fresh" and shas[0] == "sha1" and shas[2] == "sha2" and shas[50] == "sha5" and shas[9] == "sha9"
        assert s.group_attrs(9)["sample"] == ""
        s.compact(str(tmp_path / "tight.hdf5"))
        s.clear_ids([2, 3, 4242])                                      # missing ids are skipped; file attributes go (:355-367)
        assert s.get_vocab_family() is None and s.get_topk() is None
        with pytest.raises(KeyError):
            s.clear_ids([1])            # `del attrs[...]` fails there too once they are gone, after the groups went
    with DistributionStore(path, "r") as s:
        assert sorted(s.get_available_ids()) == sorted(set(data) - {1, 2, 3})
    with DistributionStore(str(tmp_path / "tight.hdf5"), "r") as t:
        assert os.path.getsize(str(tmp_path / "tight.hdf5")) < os.path.getsize(path)
        assert sorted(t.get_available_ids()) == sorted(data) and t.get_topk() == 8
        for cid, (d, i) in data.items():
            dd, ii = t.load_id(cid, storage=True)
            assert np.array_equal(_bits(dd), _bits(d)) and np.array_equal(ii, i)
        assert t.get_available_shas()[50] == "sha5"


def test_unflushed_changes_leave_the_previous_state(tmp_path):
    path = str(tmp_path / "d.hdf5")
    data = _convos(4, range(3), K=8)
    with DistributionStore(path, "w") as s:
        for cid, (d, i) in data.items():
            s.save_data(d, cid, i, content_sha="a")
    s = DistributionStore(path, "a")
    s.save_data(data[0][0], 99, data[0][1], content_sha="b")          # appended, never flushed: as after a crash
    os.close(s._fd); s._fd = None
    with DistributionStore(path, "r") as r:
        assert sorted(r.get_available_ids()) == [0, 1, 2]
        assert np.array_equal(_bits(r.load_id(1, storage=True)[0]), _bits(data[1][0]))


def test_rejects_what_it_cannot_store_or_read(tmp_path, fixture_file):
    with DistributionStore(str(tmp_path / "d.hdf5"), "w") as s:
        with pytest.raises(ValueError):
            s.save_data(np.zeros(5, np.float16), 1)
        with pytest.raises(ValueError, match="indices"):
            s.save_data(np.zeros((2, 4), np.float16), 1, np.zeros((2, 5), np.uint32))
        with pytest.raises(ValueError, match="uint32"):
            s.save_data(np.zeros((2, 4), np.float16), 1, np.full((2, 4), -1))
        s.set_dataset_attr("bad", {"a": 1})
        with pytest.raises(TypeError):
            s.flush()
        del s._file_attrs["bad"]
    with pytest.raises(F.H5FormatError, match="signature"):
        F.H5Reader(b"\0" * 4096)
    raw = bytearray(open(fixture_file, "rb").read())
    raw[8] = 2
    with pytest.raises(F.H5FormatError, match="superblock version 2"):
        F.H5Reader(bytes(raw))
    with pytest.raises(FileNotFoundError):
        DistributionStore(str(tmp_path / "absent.hdf5"), "r")


@settings(max_examples=60, deadline=None, derandomize=True)
@given(st.data())
def test_damaged_files_raise_format_errors_only(data):
    """Truncations and byte flips anywhere in a small valid file: every outcome is either a decoded
    result or H5FormatError (never another exception, never an endless walk)."""
    global _SMALL
    try:
        good = _SMALL
    except NameError:
        import tempfile
        with tempfile.TemporaryDirectory() as tmp:
            p = os.path.join(tmp, "d.hdf5")
            with DistributionStore(p, "w", chunk_bytes=128) as s:
                s.set_topk(4)
                for cid, (d, i) in _convos(5, range(12), K=4, max_rows=30).items():
                    s.save_data(d, cid, i, content_sha="x" * 8, sample="y")
            good = _SMALL = open(p, "rb").read()
    raw = bytearray(good)
    if data.draw(st.booleans()):
        raw = raw[:data.draw(st.integers(0, len(raw)))]
    for _ in range(data.draw(st.integers(0, 6))):
        if len(raw):
            raw[data.draw(st.integers(0, len(raw) - 1))] = data.draw(st.integers(0, 255))
    try:
        r = F.H5Reader(bytes(raw))
        root = r.object(r.root_address)
        r.attributes(root)
        for name, addr in r.links(root).items():
            g = r.object(addr)
            r.attributes(g)
            for _, a in r.links(g).items():
                r.read_dataset(r.object(a))
    except F.H5FormatError:
        pass


# ---------------------------------------------------------------------------------------------
# against the real library
# ---------------------------------------------------------------------------------------------
_DUMP = r"""
import h5py, numpy as np, sys
out = {}
with h5py.File(sys.argv[1], 'r') as f:
    out['__topk'] = np.asarray(f.attrs.get('topk', -1)); out['__fam'] = np.asarray(str(f.attrs.get('vocab_family')))
    for k in f:
        g = f[k]
        out['sha_' + k] = np.asarray(str(g.attrs.get('content_sha'))); out['smp_' + k] = np.asarray(str(g.attrs.get('sample')))
        if 'distributions' in g:
            assert g['distributions'].dtype == np.float16 and g['distributions'].compression == 'gzip'
            out['d_' + k] = g['distributions'][...]
        if 'indices' in g:
            assert g['indices'].dtype == np.uint32 and g['indices'].compression_opts == 6
            out['i_' + k] = g['indices'][...]
np.savez(sys.argv[2], **out)
"""


@needs_h5py
def test_libhdf5_reads_files_written_here(tmp_path):
    path, dump = str(tmp_path / "d.hdf5"), str(tmp_path / "dump.npz")
    data = _convos(6, list(range(300)) + [123456], K=24)
    with DistributionStore(path, "w", chunk_bytes=2048) as s:
        s.set_vocab_family("llama_3"); s.set_topk(24)
        for cid, (d, i) in data.items():
            s.save_data(d, cid, i, content_sha=f"{cid:064x}", sample=f"sample {cid} é中")
    with DistributionStore(path, "a") as s:                               # second session: replace and add
        data[7] = _convos(7, [7], K=24)[7]
        s.save_data(*data[7][:1], 7, data[7][1])
        s.rename_ids({8: 800})
    data[800] = data.pop(8)
    _run_h5py(_DUMP, path, dump)
    got = np.load(dump)
    assert int(got["__topk"]) == 24 and str(got["__fam"]) == "llama_3"
    assert {k[2:] for k in got.files if k.startswith("d_")} == {f"convo_{c}" for c in data}
    for cid, (d, i) in data.items():
        assert np.array_equal(_bits(got[f"d_convo_{cid}"]), _bits(d)) and np.array_equal(got[f"i_convo_{cid}"], i)
        orig = 8 if cid == 800 else cid
        assert str(got[f"sha_convo_{cid}"]) == f"{orig:064x}" and str(got[f"smp_convo_{cid}"]) == f"sample {orig} é中"


@needs_h5py
def test_appending_to_an_h5py_file_and_h5py_appending_to_ours(fixture_file, expected, tmp_path):
    dump = str(tmp_path / "dump.npz")
    add = _convos(8, [3, 5000], K=200)
    with DistributionStore(fixture_file, "a") as s:                       # ours on top of h5py's
        s.save_data(add[3][0], 3, add[3][1])
        s.save_data(add[5000][0], 5000, add[5000][1], content_sha="new", sample="n")
        s.set_topk(201)
    _run_h5py(_DUMP, fixture_file, dump)
    got = np.load(dump)
    assert int(got["__topk"]) == 201 and str(got["__fam"]) == "llama_3"
    assert np.array_equal(_bits(got["d_convo_3"]), _bits(add[3][0])) and np.array_equal(got["i_convo_5000"], add[5000][1])
    assert np.array_equal(_bits(got["d_convo_0"]), _bits(expected["d0"])) and str(got["sha_convo_3"]) == "00ff" * 16
    assert "d_convo_1000" not in got.files and str(got["sha_convo_1000"]) == f"{1000:064x}"
    # h5py on top of ours: the library's own writer must accept our groups, heaps and B-trees
    _run_h5py(r"""
import h5py, numpy as np, sys
with h5py.File(sys.argv[1], 'a') as f:
    g = f.create_group('convo_6000'); g.attrs['content_sha'] = 'lib'; g.attrs['sample'] = ''
    g.create_dataset('distributions', data=np.full((4, 200), -2.5, np.float16), compression='gzip', compression_opts=6)
    g.create_dataset('indices', data=np.arange(800, dtype=np.uint32).reshape(4, 200), compression='gzip', compression_opts=6)
    del f['convo_5000']['distributions']
    f['convo_5000'].create_dataset('distributions', data=np.zeros((2, 200), np.float16), compression='gzip', compression_opts=6)
    f['convo_5000'].attrs['content_sha'] = 'changed'
    del f['convo_1001']
""", fixture_file)
    with DistributionStore(fixture_file, "r") as s:
        ids = s.get_available_ids()
        assert 6000 in ids and 1001 not in ids and 5000 in ids
        d, i = s.load_id(6000, storage=True)
        assert (d == np.float16(-2.5)).all() and np.array_equal(i, np.arange(800, dtype=np.uint32).reshape(4, 200))
        assert s.load_id(5000, storage=True)[0].shape == (2, 200) and s.group_attrs(5000)["content_sha"] == "changed"
        assert np.array_equal(_bits(s.load_id(3, storage=True)[0]), _bits(add[3][0]))
        assert np.array_equal(s.load_id(0, storage=True)[1], expected["i0"])
