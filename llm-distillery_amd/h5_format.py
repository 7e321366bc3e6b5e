"""The subset of the HDF5 file format that a `distributions.hdf5` dataset uses, read and written
without libhdf5 (h5py is not part of this image).

What the reference stores (classes/data_manager.py:287-312, written there through h5py with its
default, oldest-compatible format): a version-0 superblock, "old style" groups (a symbol-table
message pointing at a version-1 B-tree of symbol-table nodes and a local heap of names), version-1
object headers, attributes with variable-length UTF-8 strings (kept in global heap collections) or
scalar integers, and two-dimensional chunked datasets (version-3 layout message, version-1 B-tree
of chunks) of float16 / uint32 filtered with deflate.  The reader follows the format specification
("HDF5 File Format Specification Version 3.0", sections II-IV) for exactly these structures and
refuses everything else with an H5FormatError that names what it met; the writer emits the same
structures, byte-compatible with libhdf5 1.10 (checked against the real library in the tests, where
it is installed).

Reading works on any bytes-like object (bytes, mmap).  Nothing here touches the GPU.
"""
from __future__ import annotations

import functools
import struct
import zlib
from dataclasses import dataclass, field

import numpy as np

SIGNATURE = b"\x89HDF\r\n\x1a\n"
UNDEF = 0xFFFFFFFFFFFFFFFF

MSG_NIL, MSG_DATASPACE, MSG_LINK_INFO, MSG_DATATYPE, MSG_FILL_OLD, MSG_FILL, MSG_LINK = 0, 1, 2, 3, 4, 5, 6
MSG_LAYOUT, MSG_GROUP_INFO, MSG_FILTERS, MSG_ATTRIBUTE, MSG_CONTINUATION, MSG_SYMBOL_TABLE, MSG_MTIME = 8, 10, 11, 12, 16, 17, 18
MSG_ATTRIBUTE_INFO = 21

FILTER_DEFLATE, FILTER_SHUFFLE, FILTER_FLETCHER32 = 1, 2, 3


class H5FormatError(ValueError):
    """The file is not HDF5, is damaged, or uses a feature outside the supported subset."""


def _pad8(n: int) -> int:
    return (n + 7) & ~7


# ------------------------------------------------------------------------------------------------
# datatypes
# ------------------------------------------------------------------------------------------------
@dataclass
class H5Type:
    """A parsed datatype message: `numpy` is the in-memory dtype of one element; `vlen_str` marks a
    variable-length string (element = 16-byte global-heap reference), `charset` 0 ASCII / 1 UTF-8."""
    numpy: np.dtype | None
    size: int
    vlen_str: bool = False
    fixed_str: bool = False
    charset: int = 0
    raw: bytes = b""


def parse_datatype(b: bytes) -> H5Type:
    if len(b) < 8:
        raise H5FormatError("datatype message shorter than its fixed part")
    cls, ver = b[0] & 0x0F, b[0] >> 4
    bits = b[1] | (b[2] << 8) | (b[3] << 16)
    size = struct.unpack_from("<I", b, 4)[0]
    if ver not in (1, 2, 3):
        raise H5FormatError(f"datatype message version {ver}")
    order = ">" if bits & 1 else "<"
    if cls == 0:                                           # fixed point
        bit_off, prec = struct.unpack_from("<HH", b, 8)
        if size not in (1, 2, 4, 8) or bit_off != 0 or prec != 8 * size:
            raise H5FormatError(f"integer type of {size} bytes, precision {prec}, offset {bit_off}")
        return H5Type(np.dtype(f"{order}{'i' if bits & 8 else 'u'}{size}"), size, raw=bytes(b[:12]))
    if cls == 1:                                           # floating point
        bit_off, prec, e_loc, e_size, m_loc, m_size, bias = struct.unpack_from("<HHBBBBI", b, 8)
        ieee = {2: (10, 5, 0, 10, 15), 4: (23, 8, 0, 23, 127), 8: (52, 11, 0, 52, 1023)}
        if bits & 0x40:
            raise H5FormatError("VAX byte order")
        if size not in ieee or (e_loc, e_size, m_loc, m_size, bias) != ieee[size] or bit_off != 0 or prec != 8 * size:
            raise H5FormatError(f"non-IEEE floating-point type of {size} bytes")
        return H5Type(np.dtype(f"{order}f{size}"), size, raw=bytes(b[:20]))
    if cls == 3:                                           # fixed-length string
        return H5Type(np.dtype(f"S{size}"), size, fixed_str=True, charset=(bits >> 4) & 0x0F, raw=bytes(b[:8]))
    if cls == 9:                                           # variable length
        if bits & 0x0F != 1:
            raise H5FormatError("variable-length sequence type (only variable-length strings are supported)")
        return H5Type(None, size, vlen_str=True, charset=(bits >> 8) & 0x0F, raw=bytes(b))
    raise H5FormatError(f"datatype class {cls}")


def datatype_message(dt: np.dtype) -> bytes:
    dt = np.dtype(dt)
    if dt.byteorder == ">":
        raise H5FormatError("big-endian data is not written")
    if dt.kind in "iu":
        return struct.pack("<BBBBIHH", 0x10, 0x08 if dt.kind == "i" else 0x00, 0, 0, dt.itemsize, 0, 8 * dt.itemsize)
    if dt.kind == "f":
        e_loc, e_size, m_size, bias = {2: (10, 5, 10, 15), 4: (23, 8, 23, 127), 8: (52, 11, 52, 1023)}[dt.itemsize]
        # bit field: little-endian, mantissa normalisation 2 (implied leading bit), sign bit position in byte 1
        return struct.pack("<BBBBIHHBBBBI", 0x11, 0x20, 8 * dt.itemsize - 1, 0, dt.itemsize, 0, 8 * dt.itemsize,
                           e_loc, e_size, 0, m_size, bias)
    raise H5FormatError(f"dtype {dt} is not written")


# variable-length UTF-8 string, null-terminated, over a one-byte C string base type: the message
# h5py writes for a Python `str` attribute
VLEN_UTF8_MESSAGE = struct.pack("<BBBBI", 0x19, 0x01, 0x01, 0x00, 16) + struct.pack("<BBBBI", 0x10, 0, 0, 0, 1) + \
    struct.pack("<HH", 0, 8)


# ------------------------------------------------------------------------------------------------
# reading
# ------------------------------------------------------------------------------------------------
@dataclass
class Message:
    type: int
    flags: int
    data: bytes


@dataclass
class H5Object:
    address: int
    messages: list[Message]

    def first(self, mtype: int) -> Message | None:
        for m in self.messages:
            if m.type == mtype:
                return m
        return None


@dataclass
class DatasetInfo:
    shape: tuple[int, ...]
    dtype: H5Type
    layout: int                       # 0 compact, 1 contiguous, 2 chunked
    address: int = UNDEF              # contiguous: data; chunked: B-tree
    compact: bytes = b""
    chunk: tuple[int, ...] = ()
    filters: list[tuple[int, tuple[int, ...]]] = field(default_factory=list)


def _format_errors(fn):
    """Damaged files surface as H5FormatError, whatever the parser tripped over."""
    @functools.wraps(fn)
    def wrapped(*a, **kw):
        try:
            return fn(*a, **kw)
        except H5FormatError:
            raise
        except (struct.error, IndexError, ValueError, OverflowError, UnicodeDecodeError, RecursionError, MemoryError) as e:
            raise H5FormatError(f"damaged file: {type(e).__name__}: {e}") from None
    return wrapped


class H5Reader:
    """Random access to the objects of one file image."""

    @_format_errors
    def __init__(self, buf):
        self.buf = memoryview(buf)
        self._superblock()

    # -- primitives
    def _need(self, off: int, n: int, what: str):
        if off < 0 or off + n > len(self.buf):
            raise H5FormatError(f"{what} at {off:#x}+{n} lies outside the file ({len(self.buf)} bytes)")

    def _u(self, off: int, n: int) -> int:
        self._need(off, n, "field")
        return int.from_bytes(self.buf[off:off + n], "little")

    def _superblock(self):
        base = 0
        while True:                                        # the superblock may sit at 0, 512, 1024, ...
            if base + 8 > len(self.buf):
                raise H5FormatError("no HDF5 signature")
            if bytes(self.buf[base:base + 8]) == SIGNATURE:
                break
            base = 512 if base == 0 else base * 2
        ver = self._u(base + 8, 1)
        if ver not in (0, 1):
            raise H5FormatError(f"superblock version {ver} (only the version-0/1 layout that the default "
                                "h5py settings produce is supported)")
        so, sl = self._u(base + 13, 1), self._u(base + 14, 1)
        if (so, sl) != (8, 8):
            raise H5FormatError(f"offsets of {so} and lengths of {sl} bytes")
        self.group_leaf_k, self.group_internal_k = self._u(base + 16, 2), self._u(base + 18, 2)
        p = base + 24 + (4 if ver == 1 else 0)
        self.base_address = self._u(p, 8)
        self.eof_address = self._u(p + 16, 8)
        self.root_entry_offset = p + 32
        self.superblock_offset = base
        self.eof_field_offset = p + 16
        self.root_address = self._u(p + 32 + 8, 8)
        if self.base_address != 0:
            raise H5FormatError("non-zero base address")

    # -- object headers
    @_format_errors
    def object(self, addr: int) -> H5Object:
        self._need(addr, 16, "object header")
        if bytes(self.buf[addr:addr + 4]) == b"OHDR":
            raise H5FormatError("version-2 object header (file written with libver='latest')")
        if self._u(addr, 1) != 1:
            raise H5FormatError(f"object header version {self._u(addr, 1)} at {addr:#x}")
        n_msgs, size = self._u(addr + 2, 2), self._u(addr + 8, 4)
        msgs: list[Message] = []
        blocks = [(addr + 16, size)]
        while blocks and len(msgs) < n_msgs:
            off, length = blocks.pop(0)
            self._need(off, length, "object header block")
            end = off + length
            while off + 8 <= end and len(msgs) < n_msgs:
                mtype, msize, mflags = self._u(off, 2), self._u(off + 2, 2), self._u(off + 4, 1)
                body = off + 8
                if body + msize > end:
                    raise H5FormatError(f"header message overruns its block at {off:#x}")
                if mflags & 0x02:
                    raise H5FormatError("shared header message")
                data = bytes(self.buf[body:body + msize])
                if mtype == MSG_CONTINUATION:
                    blocks.append(struct.unpack_from("<QQ", data))
                msgs.append(Message(mtype, mflags, data))
                off = body + msize
        return H5Object(addr, msgs)

    # -- groups
    def _heap_name(self, heap_addr: int, off: int) -> str:
        if bytes(self.buf[heap_addr:heap_addr + 4]) != b"HEAP":
            raise H5FormatError(f"no local heap at {heap_addr:#x}")
        size, data = self._u(heap_addr + 8, 8), self._u(heap_addr + 24, 8)
        self._need(data, size, "local heap data")
        seg = self.buf[data + off:data + size]
        n = bytes(seg).find(b"\0")
        if n < 0:
            raise H5FormatError("unterminated name in local heap")
        return bytes(seg[:n]).decode("utf-8")

    def _group_btree(self, addr: int, heap: int, out: dict[str, int], parent_level: int | None = None):
        self._need(addr, 8, "group B-tree node")
        sig = bytes(self.buf[addr:addr + 4])
        if sig == b"SNOD":
            if parent_level not in (None, 0):
                raise H5FormatError("symbol table node below an internal B-tree level")
            n = self._u(addr + 6, 2)
            for i in range(n):
                e = addr + 8 + 40 * i
                self._need(e, 40, "symbol table entry")
                if self._u(e + 16, 4) == 2:
                    raise H5FormatError("symbolic link")
                out[self._heap_name(heap, self._u(e, 8))] = self._u(e + 8, 8)
            return
        if sig != b"TREE" or self._u(addr + 4, 1) != 0:
            raise H5FormatError(f"no group B-tree node at {addr:#x}")
        level, n = self._u(addr + 5, 1), self._u(addr + 6, 2)
        if parent_level is not None and level != parent_level - 1:      # levels strictly decrease: no cycles
            raise H5FormatError(f"group B-tree node at {addr:#x} has level {level} under level {parent_level}")
        for i in range(n):
            child = self._u(addr + 24 + 8 + 16 * i, 8)       # key (8), child (8), key, child, ..., key
            if level > 0 and bytes(self.buf[child:child + 4]) != b"TREE":
                raise H5FormatError(f"level-{level} group B-tree node points at a leaf")
            self._group_btree(child, heap, out, level)

    @_format_errors
    def links(self, obj: H5Object) -> dict[str, int]:
        """name -> object header address of a group's members."""
        st = obj.first(MSG_SYMBOL_TABLE)
        if st is None:
            if obj.first(MSG_LINK_INFO) is not None or obj.first(MSG_LINK) is not None:
                raise H5FormatError("new-style group (link messages); written with libver='latest' or creation-order tracking")
            raise H5FormatError(f"object at {obj.address:#x} is not a group")
        btree, heap = struct.unpack_from("<QQ", st.data)
        out: dict[str, int] = {}
        self._group_btree(btree, heap, out)
        return out

    # -- attributes
    def _global_heap_object(self, coll: int, index: int) -> bytes:
        if bytes(self.buf[coll:coll + 4]) != b"GCOL":
            raise H5FormatError(f"no global heap collection at {coll:#x}")
        size = self._u(coll + 8, 8)
        self._need(coll, size, "global heap collection")
        off, end = coll + 16, coll + size
        while off + 16 <= end:
            idx, osize = self._u(off, 2), self._u(off + 8, 8)
            if idx == index:
                return bytes(self.buf[off + 16:off + 16 + osize])
            if idx == 0:
                break
            off += 16 + _pad8(osize)
        raise H5FormatError(f"global heap object {index} not found in collection at {coll:#x}")

    def _dataspace(self, b: bytes) -> tuple[int, ...] | None:
        ver, rank, flags = b[0], b[1], b[2]
        if ver == 1:
            off = 8
        elif ver == 2:
            if b[3] == 2:
                return None                                # null dataspace
            off = 4
        else:
            raise H5FormatError(f"dataspace message version {ver}")
        return tuple(struct.unpack_from(f"<{rank}Q", b, off)) if rank else ()

    def _decode_elements(self, t: H5Type, shape, raw: bytes):
        count = int(np.prod(shape)) if shape else 1
        if t.vlen_str:
            vals = []
            for i in range(count):
                length, coll, idx = struct.unpack_from("<IQI", raw, 16 * i)
                vals.append("" if coll == 0 and idx == 0 else
                            self._global_heap_object(coll, idx)[:length].decode("utf-8"))
            return vals[0] if shape == () else np.array(vals, dtype=object).reshape(shape)
        arr = np.frombuffer(raw, dtype=t.numpy, count=count)
        if t.fixed_str:
            vals = [bytes(x).rstrip(b"\0") for x in arr]
            vals = [v.decode("utf-8") if t.charset == 1 else v for v in vals]
            return vals[0] if shape == () else np.array(vals, dtype=object).reshape(shape)
        arr = arr.astype(t.numpy.newbyteorder("="))
        return arr[0] if shape == () else arr.reshape(shape)

    @_format_errors
    def attributes(self, obj: H5Object) -> dict[str, object]:
        out: dict[str, object] = {}
        for m in obj.messages:
            if m.type != MSG_ATTRIBUTE:
                continue
            b = m.data
            ver = b[0]
            nsz, tsz, ssz = struct.unpack_from("<HHH", b, 2)
            if ver == 1:
                off = 8
                name = b[off:off + nsz]; off += _pad8(nsz)
                tmsg = b[off:off + tsz]; off += _pad8(tsz)
                smsg = b[off:off + ssz]; off += _pad8(ssz)
            elif ver in (2, 3):
                if b[1] & 0x03:
                    raise H5FormatError("attribute with shared datatype or dataspace")
                off = 8 + (1 if ver == 3 else 0)
                name = b[off:off + nsz]; off += nsz
                tmsg = b[off:off + tsz]; off += tsz
                smsg = b[off:off + ssz]; off += ssz
            else:
                raise H5FormatError(f"attribute message version {ver}")
            shape = self._dataspace(smsg)
            key = name.split(b"\0")[0].decode("utf-8")
            out[key] = None if shape is None else self._decode_elements(parse_datatype(tmsg), shape, b[off:])
        info = obj.first(MSG_ATTRIBUTE_INFO)
        if info is not None:                               # version, flags, [max creation index], fractal heap address, ...
            heap = struct.unpack_from("<Q", info.data, 2 + (2 if info.data[1] & 1 else 0))[0]
            if heap != UNDEF:
                raise H5FormatError("attributes in dense storage (fractal heap)")
        return out

    # -- datasets
    @_format_errors
    def dataset_info(self, obj: H5Object) -> DatasetInfo:
        sp, ty, lay = obj.first(MSG_DATASPACE), obj.first(MSG_DATATYPE), obj.first(MSG_LAYOUT)
        if sp is None or ty is None or lay is None:
            raise H5FormatError(f"object at {obj.address:#x} is not a dataset")
        shape = self._dataspace(sp.data)
        if shape is None:
            raise H5FormatError("dataset with a null dataspace")
        t = parse_datatype(ty.data)
        if t.numpy is None or t.fixed_str:
            raise H5FormatError("dataset of strings")
        b = lay.data
        if b[0] != 3:
            raise H5FormatError(f"data layout message version {b[0]}")
        info = DatasetInfo(shape, t, b[1])
        if b[1] == 0:
            n = struct.unpack_from("<H", b, 2)[0]
            info.compact = b[4:4 + n]
        elif b[1] == 1:
            info.address = struct.unpack_from("<Q", b, 2)[0]
        elif b[1] == 2:
            nd = b[2]
            info.address = struct.unpack_from("<Q", b, 3)[0]
            dims = struct.unpack_from(f"<{nd}I", b, 11)
            if nd != len(shape) + 1 or dims[-1] != t.size:
                raise H5FormatError("chunk dimensionality does not match the dataspace")
            info.chunk = tuple(dims[:-1])
        else:
            raise H5FormatError(f"data layout class {b[1]}")
        fm = obj.first(MSG_FILTERS)
        if fm is not None:
            info.filters = _parse_filters(fm.data)
        return info

    def _chunks(self, addr: int, nd: int, out: list, parent_level: int | None = None):
        if addr == UNDEF:
            return
        self._need(addr, 24, "chunk B-tree node")
        if bytes(self.buf[addr:addr + 4]) != b"TREE" or self._u(addr + 4, 1) != 1:
            raise H5FormatError(f"no chunk B-tree node at {addr:#x}")
        level, n = self._u(addr + 5, 1), self._u(addr + 6, 2)
        if parent_level is not None and level != parent_level - 1:      # levels strictly decrease: no cycles
            raise H5FormatError(f"chunk B-tree node at {addr:#x} has level {level} under level {parent_level}")
        ksz = 8 + 8 * (nd + 1)
        off = addr + 24
        self._need(off, n * (ksz + 8) + ksz, "chunk B-tree entries")
        for _ in range(n):
            nbytes, mask = struct.unpack_from("<II", self.buf, off)
            offs = struct.unpack_from(f"<{nd}Q", self.buf, off + 8)
            child = self._u(off + ksz, 8)
            if level == 0:
                out.append((offs, nbytes, mask, child))
            else:
                self._chunks(child, nd, out, level)
            off += ksz + 8

    @_format_errors
    def read_dataset(self, obj: H5Object, info: DatasetInfo | None = None, out: np.ndarray | None = None) -> np.ndarray:
        """The whole dataset in its stored dtype (native byte order); decoded into `out` (same shape,
        itemsize and kind, e.g. a view of pinned memory) when given."""
        info = info or self.dataset_info(obj)
        dt, shape = info.dtype.numpy, info.shape
        native = dt.newbyteorder("=")
        count = int(np.prod(shape)) if shape else 1
        if count * dt.itemsize > 1100 * len(self.buf) + (1 << 20):      # deflate expands at most ~1032 times
            raise H5FormatError(f"dataset of {shape} {native} cannot come from a file of {len(self.buf)} bytes")
        if out is not None and (tuple(out.shape) != tuple(shape) or out.dtype.itemsize != dt.itemsize):
            raise ValueError(f"destination {out.shape} {out.dtype} for a dataset {shape} {native}")
        if out is None:
            out = np.zeros(shape, dtype=native)
            fresh = True
        else:
            out = out.view(native) if out.dtype != native else out
            fresh = False
        if info.layout == 0:
            out[...] = np.frombuffer(info.compact, dtype=dt, count=count).reshape(shape)
            return out
        if info.layout == 1:
            if info.address == UNDEF:
                out[...] = 0
                return out
            self._need(info.address, count * dt.itemsize, "contiguous dataset")
            out[...] = np.frombuffer(self.buf, dtype=dt, count=count, offset=info.address).reshape(shape)
            return out
        if count == 0:
            return out
        if not fresh:
            out[...] = 0                                   # chunks that were never written read as the fill value
        for chunk in self.chunk_list(info):
            self.decode_chunk(info, chunk, out)
        return out

    @_format_errors
    def chunk_list(self, info: DatasetInfo) -> list:
        """The stored chunks of a chunked dataset: (offsets, stored bytes, filter mask, address)."""
        chunks: list = []
        if info.layout == 2:
            self._chunks(info.address, len(info.shape), chunks)
        return chunks

    @_format_errors
    def decode_chunk(self, info: DatasetInfo, chunk, out: np.ndarray):
        """Undo the filters of one chunk and copy its part inside the dataspace into `out` (an array
        of the dataset's shape, zero where no chunk is stored).  Chunks are independent: callers
        may decode them on several threads."""
        offs, nbytes, mask, addr = chunk
        dt, shape = info.dtype.numpy, info.shape
        csize = int(np.prod(info.chunk)) * dt.itemsize
        self._need(addr, nbytes, "chunk")
        raw = _unfilter(bytes(self.buf[addr:addr + nbytes]), info.filters, mask, dt.itemsize, csize + 4)
        if len(raw) != csize:
            raise H5FormatError(f"chunk at {addr:#x} decodes to {len(raw)} bytes, expected {csize}")
        if any(o >= s for o, s in zip(offs, shape)):
            raise H5FormatError("chunk outside the dataspace")
        block = np.frombuffer(raw, dtype=dt).reshape(info.chunk)
        sel_out = tuple(slice(o, min(o + c, s)) for o, c, s in zip(offs, info.chunk, shape))
        sel_in = tuple(slice(0, s.stop - s.start) for s in sel_out)
        out[sel_out] = block[sel_in]


def _parse_filters(b: bytes) -> list[tuple[int, tuple[int, ...]]]:
    ver, n = b[0], b[1]
    out = []
    if ver == 1:
        off = 8
        for _ in range(n):
            fid, nlen, _flags, ncd = struct.unpack_from("<HHHH", b, off)
            off += 8 + _pad8(nlen)
            cd = struct.unpack_from(f"<{ncd}I", b, off)
            off += 4 * ncd + (4 if ncd % 2 else 0)
            out.append((fid, cd))
    elif ver == 2:
        off = 2
        for _ in range(n):
            fid = struct.unpack_from("<H", b, off)[0]; off += 2
            nlen = 0
            if fid >= 256:
                nlen = struct.unpack_from("<H", b, off)[0]; off += 2
            _flags, ncd = struct.unpack_from("<HH", b, off); off += 4 + nlen
            cd = struct.unpack_from(f"<{ncd}I", b, off); off += 4 * ncd
            out.append((fid, cd))
    else:
        raise H5FormatError(f"filter pipeline message version {ver}")
    for fid, _ in out:
        if fid not in (FILTER_DEFLATE, FILTER_SHUFFLE, FILTER_FLETCHER32):
            raise H5FormatError(f"filter {fid} (supported: deflate, shuffle, fletcher32)")
    return out


def _unfilter(raw: bytes, filters, mask: int, itemsize: int, limit: int) -> bytes:
    for i in range(len(filters) - 1, -1, -1):              # undo the pipeline last filter first
        if mask & (1 << i):
            continue
        fid = filters[i][0]
        if fid == FILTER_DEFLATE:
            try:
                d = zlib.decompressobj()
                raw = d.decompress(raw, limit)
                if d.unconsumed_tail:
                    raise H5FormatError(f"chunk inflates beyond its {limit} bytes")
            except zlib.error as e:
                raise H5FormatError(f"damaged deflate stream: {e}") from None
        elif fid == FILTER_FLETCHER32:
            raw = raw[:-4]
        elif fid == FILTER_SHUFFLE:
            n = len(raw) // itemsize
            body = np.frombuffer(raw, dtype=np.uint8, count=n * itemsize).reshape(itemsize, n).T
            raw = np.ascontiguousarray(body).tobytes() + raw[n * itemsize:]
    return raw


# ------------------------------------------------------------------------------------------------
# writing: building blocks.  Every function returns bytes for a structure whose own address is
# given where the structure refers to itself or to neighbours placed by the caller.
# ------------------------------------------------------------------------------------------------
def _message(mtype: int, body: bytes, flags: int = 0) -> bytes:
    body = body + b"\0" * (_pad8(len(body)) - len(body))
    return struct.pack("<HHB3x", mtype, len(body), flags) + body


def object_header(messages: list[bytes]) -> bytes:
    body = b"".join(messages)
    # version 1, one reference; 4 bytes of padding align the first message to 8
    return struct.pack("<BxHII4x", 1, len(messages), 1, len(body)) + body


def dataspace_message(shape: tuple[int, ...]) -> bytes:
    rank = len(shape)
    body = struct.pack("<BBB5x", 1, rank, 1 if rank else 0)
    if rank:
        body += struct.pack(f"<{rank}Q", *shape) * 2        # dimensions, then maximum dimensions
    return _message(MSG_DATASPACE, body)


def attribute_message(name: str, type_msg: bytes, shape: tuple[int, ...], data: bytes) -> bytes:
    nm = name.encode("utf-8") + b"\0"
    space = dataspace_message(shape)[8:]
    def pad(x):
        return x + b"\0" * (_pad8(len(x)) - len(x))
    body = struct.pack("<BxHHH", 1, len(nm), len(type_msg), len(space)) + pad(nm) + pad(type_msg) + pad(space) + data
    return _message(MSG_ATTRIBUTE, body)


def global_heap_collection(objects: list[bytes]) -> bytes:
    """One collection holding `objects` as heap objects 1..n (then the free-space object 0)."""
    body = b""
    for i, o in enumerate(objects, start=1):
        body += struct.pack("<HH4xQ", i, 0, len(o)) + o + b"\0" * (_pad8(len(o)) - len(o))
    size = max(4096, _pad8(16 + len(body) + 16))
    free = size - 16 - len(body)
    body += struct.pack("<HH4xQ", 0, 0, free) + b"\0" * (free - 16)    # the free-space object counts its own header
    return b"GCOL" + struct.pack("<B3xQ", 1, size) + body


def btree_nodes(node_type: int, keys: list[bytes], children: list[int], last_key: bytes, k: int, base: int):
    """A version-1 B-tree over `children` (addresses, in key order) with `keys[i]` the left key of
    child i and `last_key` closing the rightmost child.  Nodes hold at most 2k children and are
    laid out from address `base`; returns (bytes, root address).  Every node is written at its full
    size (2k entries), as libhdf5 does."""
    ksz = len(last_key)
    node_bytes = 24 + (2 * k + 1) * ksz + 2 * k * 8
    out = bytearray()
    level = 0
    cur_keys, cur_children = list(keys), list(children)
    cur_last = last_key
    while True:
        groups = [(i, min(i + 2 * k, len(cur_children))) for i in range(0, max(len(cur_children), 1), 2 * k)]
        addrs = [base + len(out) + j * node_bytes for j in range(len(groups))]
        next_keys, next_children = [], []
        for j, (lo, hi) in enumerate(groups):
            left = addrs[j - 1] if j > 0 else UNDEF
            right = addrs[j + 1] if j + 1 < len(groups) else UNDEF
            node = bytearray(b"TREE" + struct.pack("<BBHQQ", node_type, level, hi - lo, left, right))
            for i in range(lo, hi):
                node += cur_keys[i] + struct.pack("<Q", cur_children[i])
            node += cur_keys[hi] if hi < len(cur_children) else cur_last
            node += b"\0" * (node_bytes - len(node))
            out += node
            next_keys.append(cur_keys[lo] if cur_children else cur_last)
            next_children.append(addrs[j])
        if len(groups) == 1:
            return bytes(out), addrs[0]
        cur_keys, cur_children = next_keys, next_children
        level += 1


def chunked_dataset(arr: np.ndarray, base: int, level: int = 6, chunk_bytes: int = 1 << 20) -> tuple[bytes, int]:
    """A two-dimensional dataset, chunked by whole rows and deflated: (bytes, object header
    address).  Everything the dataset owns (chunks, chunk B-tree, object header) is laid out from
    address `base`."""
    if arr.ndim != 2:
        raise H5FormatError("datasets are two-dimensional [rows, width]")
    arr = np.ascontiguousarray(arr)
    dt = arr.dtype
    rows, width = arr.shape
    per = max(1, min(max(rows, 1), chunk_bytes // max(1, width * dt.itemsize)))
    out = bytearray()
    keys, children = [], []
    for r0 in range(0, rows, per):
        block = arr[r0:r0 + per]
        if block.shape[0] < per:                           # edge chunks are stored at full size
            block = np.concatenate([block, np.zeros((per - block.shape[0], width), dtype=dt)])
        z = zlib.compress(block.tobytes(), level)
        keys.append(struct.pack("<IIQQQ", len(z), 0, r0, 0, 0))
        children.append(base + len(out))
        out += z + b"\0" * (_pad8(len(z)) - len(z))
    btree_addr = UNDEF
    if children:
        last = struct.pack("<IIQQQ", 0, 0, (rows + per - 1) // per * per, width, 0)
        tree, btree_addr = btree_nodes(1, keys, children, last, 32, base + len(out))
        out += tree
    header_addr = base + len(out)
    layout = struct.pack("<BBBQIII", 3, 2, 3, btree_addr, per, max(width, 1), dt.itemsize)
    filters = struct.pack("<BB6x", 1, 1) + struct.pack("<HHHH", FILTER_DEFLATE, 8, 1, 1) + b"deflate\0" + struct.pack("<II", level, 0)
    out += object_header([
        dataspace_message((rows, width)),
        _message(MSG_DATATYPE, datatype_message(dt), flags=1),
        _message(MSG_FILL, struct.pack("<BBBBI", 2, 3, 0, 1, 0), flags=1),  # allocate incrementally, default (zero) fill
        _message(MSG_FILTERS, filters, flags=1),
        _message(MSG_LAYOUT, layout),
    ])
    out += b"\0" * (_pad8(len(out)) - len(out))
    return bytes(out), header_addr


def group_structures(members: dict[str, int], base: int, leaf_k: int = 4, internal_k: int = 16) -> tuple[bytes, int, int]:
    """Local heap, symbol-table nodes and B-tree of an old-style group: (bytes, B-tree address,
    heap address), laid out from `base`."""
    names = sorted(members, key=lambda s: s.encode("utf-8"))
    heap_data = bytearray(b"\0" * 8)                        # offset 0: the empty name that keys the leftmost child
    offsets = {}
    for n in names:
        offsets[n] = len(heap_data)
        e = n.encode("utf-8") + b"\0"
        heap_data += e + b"\0" * (_pad8(len(e)) - len(e))
    free_off = len(heap_data)
    heap_data += struct.pack("<QQ", 1, 16)                  # one free block: next = 1 (none), size 16
    out = bytearray()
    heap_addr = base
    out += b"HEAP" + struct.pack("<B3xQQQ", 0, len(heap_data), free_off, heap_addr + 32) + heap_data
    snod_bytes = 8 + 2 * leaf_k * 40
    keys, children = [], []
    for i in range(0, len(names), 2 * leaf_k):
        part = names[i:i + 2 * leaf_k]
        node = bytearray(b"SNOD" + struct.pack("<BxH", 1, len(part)))
        for n in part:
            node += struct.pack("<QQI4x16x", offsets[n], members[n], 0)
        node += b"\0" * (snod_bytes - len(node))
        keys.append(struct.pack("<Q", offsets[names[i - 1]] if i else 0))
        children.append(base + len(out))
        out += node
    last = struct.pack("<Q", offsets[names[-1]] if names else 0)
    tree, btree_addr = btree_nodes(0, keys, children, last, internal_k, base + len(out))
    out += tree
    return bytes(out), btree_addr, heap_addr


def superblock(root_header: int, root_btree: int, root_heap: int, eof: int, leaf_k: int = 4, internal_k: int = 16) -> bytes:
    sb = SIGNATURE + struct.pack("<BBBxBBBxHHI", 0, 0, 0, 0, 8, 8, leaf_k, internal_k, 0)
    sb += struct.pack("<QQQQ", 0, UNDEF, eof, UNDEF)
    sb += struct.pack("<QQI4xQQ", 0, root_header, 1, root_btree, root_heap)
    return sb
