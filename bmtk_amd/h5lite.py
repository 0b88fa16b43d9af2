"""A small reader and writer for the subset of HDF5 that SONATA files use.

The reference reads and writes its network, input and output files with h5py
(bmtk/utils/sonata/population.py:349-456, bmtk/utils/reports/spike_trains/
spikes_file_writers.py:35-73, spike_train_readers.py:93-292).  h5py is not part
of this image, so the files are handled directly, following the published
"HDF5 File Format Specification Version 3.0".

Reader: superblock 0/1 (and 2/3 for the root address), version-1 and
version-2 object headers, symbol-table groups (version-1 B-trees + local
heaps) and compact link messages, dataspace 1/2, datatypes fixed-point,
floating-point, fixed strings, variable-length strings (global heap), enums over
integers (h5py booleans) and compounds of those, layouts compact / contiguous /
chunked (version-1 chunk B-tree) with the deflate and shuffle filters, attribute
messages 1-3.

Writer: the "earliest" layout h5py itself produces by default — superblock 0,
symbol-table groups, version-1 object headers, contiguous little-endian numeric
datasets, fixed-length string attributes and numeric attributes.

`File(path)` gives a read-only tree: `f["/edges/v1_to_v1/source_node_id"][()]`
returns a numpy array, `.attrs` a dict, groups iterate over member names.
"""
from __future__ import annotations

import mmap
import struct
import zlib

import numpy as np

SIGNATURE = b"\x89HDF\r\n\x1a\n"
UNDEF = 0xFFFFFFFFFFFFFFFF


class H5Error(ValueError):
    pass


# ----------------------------------------------------------------------------------------------------------------
# reading
# ----------------------------------------------------------------------------------------------------------------

def _u(buf, off, size):
    return int.from_bytes(buf[off:off + size], "little")


class _Datatype:
    """A parsed datatype message: `dtype` is the numpy dtype of one element, `vlen_str` marks variable-length
    strings (16-byte global-heap references in the file), `size` the element size in the file."""

    def __init__(self, dtype, size, vlen_str=False, is_bool=False):
        self.dtype = dtype
        self.size = size
        self.vlen_str = vlen_str
        self.is_bool = is_bool


def _parse_datatype(buf, off):
    """-> (_Datatype, bytes consumed)."""
    cls_ver = buf[off]
    cls, bits0, bits1 = cls_ver & 0x0F, buf[off + 1], buf[off + 2]
    size = _u(buf, off + 4, 4)
    p = off + 8
    if cls == 0:  # fixed point
        order = ">" if bits0 & 1 else "<"
        kind = "i" if bits0 & 8 else "u"
        return _Datatype(np.dtype(f"{order}{kind}{size}"), size), 8 + 4
    if cls == 1:  # floating point
        order = ">" if bits0 & 1 else "<"
        return _Datatype(np.dtype(f"{order}f{size}"), size), 8 + 12
    if cls == 3:  # fixed-length string
        return _Datatype(np.dtype(f"S{size}"), size), 8
    if cls == 9:  # variable length
        base, used = _parse_datatype(buf, p)
        if (bits0 & 0x0F) != 1:
            raise H5Error("variable-length sequences other than strings are not supported")
        return _Datatype(np.dtype("O"), size, vlen_str=True), 8 + used
    if cls == 8:  # enumeration (h5py stores bool as an enum over int8)
        base, used = _parse_datatype(buf, p)
        n = bits0 | (bits1 << 8)
        q = p + used
        names = []
        for _ in range(n):
            end = buf.find(b"\0", q)
            names.append(bytes(buf[q:end]))
            q += ((end - q) // 8 + 1) * 8 if (cls_ver >> 4) < 3 else end - q + 1
        q += n * base.size
        return _Datatype(base.dtype, size, is_bool=sorted(names) == [b"FALSE", b"TRUE"]), q - off
    if cls == 6:  # compound
        version = cls_ver >> 4
        n = bits0 | (bits1 << 8)
        q = p
        fields = []
        for _ in range(n):
            end = buf.find(b"\0", q)
            name = bytes(buf[q:end]).decode()
            if version < 3:
                q += ((end - q) // 8 + 1) * 8
            else:
                q = end + 1
            if version == 1:
                moff = _u(buf, q, 4)
                q += 4 + 1 + 3 + 4 + 4 + 16
            elif version == 2:
                moff = _u(buf, q, 4)
                q += 4
            else:
                nb = max(1, (size.bit_length() + 7) // 8)
                moff = _u(buf, q, nb)
                q += nb
            member, used = _parse_datatype(buf, q)
            if member.vlen_str:
                raise H5Error("compound members of variable length are not supported")
            q += used
            fields.append((name, member.dtype, moff))
        dt = np.dtype({"names": [f[0] for f in fields], "formats": [f[1] for f in fields],
                       "offsets": [f[2] for f in fields], "itemsize": size})
        return _Datatype(dt, size), q - off
    raise H5Error(f"datatype class {cls} is not supported")


def _parse_dataspace(buf, off):
    version, rank, flags = buf[off], buf[off + 1], buf[off + 2]
    if version == 1:
        p = off + 8
    elif version == 2:
        if buf[off + 3] == 2:  # null dataspace
            return None
        p = off + 4
    else:
        raise H5Error(f"dataspace version {version}")
    return tuple(_u(buf, p + 8 * i, 8) for i in range(rank))


class _Object:
    """One object header, parsed into its messages."""

    def __init__(self, f, addr):
        self.f = f
        self.addr = addr
        self.msgs = []  # (type, offset of the data in f.buf, size)
        buf = f.buf
        if buf[addr:addr + 4] == b"OHDR":
            self._read_v2(addr)
        else:
            if buf[addr] != 1:
                raise H5Error(f"object header version {buf[addr]} at {addr}")
            nmsg = _u(buf, addr + 2, 2)
            size = _u(buf, addr + 8, 4)
            self._read_v1_block(addr + 16, size, nmsg)

    def _read_v1_block(self, start, size, nmsg):
        buf = self.f.buf
        blocks = [(start, size)]
        while blocks and len(self.msgs) < nmsg:
            p, left = blocks.pop(0)
            end = p + left
            while p + 8 <= end and len(self.msgs) < nmsg:
                mtype, msize = _u(buf, p, 2), _u(buf, p + 2, 2)
                data = p + 8
                self.msgs.append((mtype, data, msize))
                if mtype == 0x10:
                    blocks.append((_u(buf, data, 8), _u(buf, data + 8, 8)))
                p = data + msize

    def _read_v2(self, addr):
        buf = self.f.buf
        flags = buf[addr + 5]
        p = addr + 6
        if flags & 0x20:
            p += 16
        if flags & 0x10:
            p += 4
        nb = 1 << (flags & 3)
        chunk0 = _u(buf, p, nb)
        p += nb
        blocks = [(p, chunk0)]
        track = bool(flags & 0x04)
        while blocks:
            p, left = blocks.pop(0)
            end = p + left
            while p + 4 + (2 if track else 0) <= end:
                mtype, msize = buf[p], _u(buf, p + 1, 2)
                data = p + 4 + (2 if track else 0)
                if data + msize > end:
                    break
                self.msgs.append((mtype, data, msize))
                if mtype == 0x10:
                    caddr, clen = _u(buf, data, 8), _u(buf, data + 8, 8)
                    blocks.append((caddr + 4, clen - 8))  # skip "OCHK", drop the checksum
                p = data + msize

    def find(self, mtype):
        return [(d, s) for t, d, s in self.msgs if t == mtype]


class _Attrs(dict):
    pass


def _read_vlen_strings(f, raw, count):
    out = []
    for i in range(count):
        rec = raw[16 * i:16 * i + 16]
        length = _u(rec, 0, 4)
        gaddr, index = _u(rec, 4, 8), _u(rec, 12, 4)
        out.append(f._global_heap_object(gaddr, index)[:length].decode("utf-8", "replace") if length else "")
    return out


def _decode(f, dt, shape, raw):
    count = int(np.prod(shape)) if shape else 1
    if dt.vlen_str:
        vals = _read_vlen_strings(f, raw, count)
        if shape == ():
            return vals[0]
        return np.array(vals, dtype=object).reshape(shape)
    arr = np.frombuffer(raw, dtype=dt.dtype, count=count).reshape(shape).copy()  # detach from the mapping
    if dt.is_bool:
        arr = arr.astype(bool)
    if dt.dtype.kind == "S" and shape == ():
        return bytes(arr[()]).split(b"\0")[0].decode("utf-8", "replace")
    return arr[()] if shape == () else arr


class _Node:
    def __init__(self, f, obj, name):
        self._f = f
        self._obj = obj
        self.name = name
        self._attrs = None

    @property
    def attrs(self):
        if self._attrs is None:
            self._attrs = _Attrs()
            buf = self._f.buf
            for d, s in self._obj.find(0x0C):
                version = buf[d]
                nsize, tsize, ssize = _u(buf, d + 2, 2), _u(buf, d + 4, 2), _u(buf, d + 6, 2)
                p = d + 8 + (1 if version == 3 else 0)
                pad = (lambda n: (n + 7) // 8 * 8) if version == 1 else (lambda n: n)
                name = bytes(buf[p:p + nsize]).split(b"\0")[0].decode()
                p += pad(nsize)
                dt, _ = _parse_datatype(buf, p)
                p += pad(tsize)
                shape = _parse_dataspace(buf, p)
                p += pad(ssize)
                if shape is None:
                    self._attrs[name] = None
                    continue
                count = int(np.prod(shape)) if shape else 1
                self._attrs[name] = _decode(self._f, dt, shape, bytes(buf[p:p + count * dt.size]))
        return self._attrs


class Dataset(_Node):
    def __init__(self, f, obj, name):
        super().__init__(f, obj, name)
        buf = f.buf
        (d, _), = obj.find(0x03)
        self._dt, _ = _parse_datatype(buf, d)
        (d, _), = obj.find(0x01)
        shape = _parse_dataspace(buf, d)
        self.shape = () if shape is None else shape
        self.dtype = np.dtype(bool) if self._dt.is_bool else self._dt.dtype

    def __len__(self):
        return self.shape[0]

    @property
    def size(self):
        return int(np.prod(self.shape)) if self.shape else 1

    def _raw(self):
        f, buf = self._f, self._f.buf
        (d, s), = self._obj.find(0x08)
        version, nbytes = buf[d], self.size * self._dt.size
        if version != 3:
            raise H5Error(f"data layout version {version}")
        cls = buf[d + 1]
        if cls == 0:
            n = _u(buf, d + 2, 2)
            return bytes(buf[d + 4:d + 4 + n])
        if cls == 1:
            addr = _u(buf, d + 2, 8)
            if addr == UNDEF:
                return bytes(nbytes)
            return memoryview(buf)[addr:addr + nbytes]  # no copy: the file is memory-mapped
        if cls == 2:
            rank = buf[d + 2]
            btree = _u(buf, d + 3, 8)
            cdims = [_u(buf, d + 11 + 4 * i, 4) for i in range(rank)]
            return self._read_chunks(btree, cdims[:-1], cdims[-1])
        raise H5Error(f"data layout class {cls}")

    def _filters(self):
        buf = self._f.buf
        out = []
        for d, s in self._obj.find(0x0B):
            version, n = buf[d], buf[d + 1]
            p = d + (8 if version == 1 else 2)
            for _ in range(n):
                fid = _u(buf, p, 2)
                if version == 1 or fid >= 256:
                    nlen = _u(buf, p + 2, 2)
                    p += 2
                else:
                    nlen = 0
                ncd = _u(buf, p + 4, 2)
                p += 6
                p += (nlen + 7) // 8 * 8 if version == 1 else nlen
                cd = [_u(buf, p + 4 * i, 4) for i in range(ncd)]
                p += 4 * ncd
                if version == 1 and ncd % 2:
                    p += 4
                out.append((fid, cd))
        return out

    def _read_chunks(self, btree, cdims, esize):
        f, buf = self._f, self._f.buf
        shape = self.shape
        rank = len(shape)
        filters = self._filters()
        out = np.zeros(shape, dtype=np.dtype((np.void, esize)))
        if btree == UNDEF:
            return out.tobytes()

        def walk(addr):
            if buf[addr:addr + 4] != b"TREE" or buf[addr + 4] != 1:
                raise H5Error("bad chunk B-tree node")
            level, used = buf[addr + 5], _u(buf, addr + 6, 2)
            p = addr + 24
            ksz = 8 + 8 * (rank + 1)
            for _ in range(used):
                csize, mask = _u(buf, p, 4), _u(buf, p + 4, 4)
                offs = [_u(buf, p + 8 + 8 * i, 8) for i in range(rank)]
                child = _u(buf, p + ksz, 8)
                p += ksz + 8
                if level > 0:
                    walk(child)
                    continue
                data = bytes(buf[child:child + csize])
                for k, (fid, cd) in reversed(list(enumerate(filters))):
                    if mask & (1 << k):
                        continue
                    if fid == 1:
                        data = zlib.decompress(data)
                    elif fid == 2:
                        n = len(data) // esize
                        data = np.frombuffer(data, np.uint8).reshape(esize, n).T.tobytes()
                    elif fid == 3:
                        data = data[:-4]  # fletcher32 checksum, not verified
                    else:
                        raise H5Error(f"filter {fid} is not supported")
                chunk = np.frombuffer(data, dtype=out.dtype, count=int(np.prod(cdims))).reshape(cdims)
                sl_out = tuple(slice(o, min(o + c, s)) for o, c, s in zip(offs, cdims, shape))
                sl_in = tuple(slice(0, s.stop - s.start) for s in sl_out)
                out[sl_out] = chunk[sl_in]

        walk(btree)
        return out.tobytes()

    def __getitem__(self, key):
        arr = _decode(self._f, self._dt, self.shape, self._raw())
        if key is Ellipsis or key == ():
            return arr
        return arr[key]

    def __array__(self, dtype=None, copy=None):
        a = self[()]
        return a if dtype is None else a.astype(dtype)


class Group(_Node):
    def __init__(self, f, obj, name):
        super().__init__(f, obj, name)
        self._links = None

    def _load(self):
        if self._links is not None:
            return
        f, buf = self._f, self._f.buf
        links = {}
        for d, s in self._obj.find(0x11):  # symbol table
            btree, heap = _u(buf, d, 8), _u(buf, d + 8, 8)
            if buf[heap:heap + 4] != b"HEAP":
                raise H5Error("bad local heap")
            hdata = _u(buf, heap + 24, 8)

            def walk(addr):
                if buf[addr:addr + 4] == b"SNOD":
                    n = _u(buf, addr + 6, 2)
                    for i in range(n):
                        e = addr + 8 + 40 * i
                        noff, oaddr = _u(buf, e, 8), _u(buf, e + 8, 8)
                        end = buf.find(b"\0", hdata + noff)
                        links[bytes(buf[hdata + noff:end]).decode()] = oaddr
                    return
                if buf[addr:addr + 4] != b"TREE" or buf[addr + 4] != 0:
                    raise H5Error("bad group B-tree node")
                used = _u(buf, addr + 6, 2)
                p = addr + 24
                for i in range(used):
                    walk(_u(buf, p + 8 + 16 * i, 8))

            walk(btree)
        for d, s in self._obj.find(0x06):  # link message (compact new-style groups)
            version, flags = buf[d], buf[d + 1]
            p = d + 2
            ltype = 0
            if flags & 0x08:
                ltype = buf[p]
                p += 1
            if flags & 0x04:
                p += 8
            if flags & 0x10:
                p += 1
            nb = 1 << (flags & 3)
            nlen = _u(buf, p, nb)
            p += nb
            name = bytes(buf[p:p + nlen]).decode()
            p += nlen
            if ltype == 0:
                links[name] = _u(buf, p, 8)
        if self._obj.find(0x02) and not links:
            (d, s), = self._obj.find(0x02)
            if _u(buf, d + 2 + (8 if buf[d + 1] & 1 else 0), 8) != UNDEF:
                raise H5Error("dense (fractal-heap) groups are not supported")
        self._links = links

    def keys(self):
        self._load()
        return sorted(self._links)

    def __iter__(self):
        return iter(self.keys())

    def __len__(self):
        return len(self.keys())

    def __contains__(self, path):
        try:
            self[path]
            return True
        except KeyError:
            return False

    def items(self):
        return [(k, self[k]) for k in self.keys()]

    def __getitem__(self, path):
        node = self
        if path.startswith("/"):
            node = self._f.root
        for part in [p for p in path.split("/") if p]:
            if not isinstance(node, Group):
                raise KeyError(path)
            node._load()
            if part not in node._links:
                raise KeyError(path)
            node = self._f._node(node._links[part], node.name.rstrip("/") + "/" + part)
        return node


class File(Group):
    """Read-only view of a memory-mapped HDF5 file: a data set is read from disk when it is asked for, so a
    multi-gigabyte edge file costs the memory of the arrays taken from it and no more."""

    def __init__(self, path, mode="r"):
        if mode != "r":
            raise H5Error("File() reads; use h5lite.write() to create a file")
        self.path = str(path)
        self._fh = open(path, "rb")
        try:
            self.buf = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError:
            self._fh.close()
            raise H5Error(f"{path}: not an HDF5 file")
        buf = self.buf
        base = 0
        while buf[base:base + 8] != SIGNATURE:
            base = 512 if base == 0 else base * 2
            if base >= len(buf):
                raise H5Error(f"{path}: not an HDF5 file")
        if base:
            raise H5Error("files with a user block are not supported")
        version = buf[8]
        if version in (0, 1):
            if buf[13] != 8 or buf[14] != 8:
                raise H5Error("only 8-byte offsets and lengths are supported")
            p = 24 + (4 if version == 1 else 0) + 32
            root_addr = _u(buf, p + 8, 8)
        elif version in (2, 3):
            if buf[9] != 8 or buf[10] != 8:
                raise H5Error("only 8-byte offsets and lengths are supported")
            root_addr = _u(buf, 12 + 24, 8)
        else:
            raise H5Error(f"superblock version {version}")
        self._cache = {}
        self._gheaps = {}
        self.root = self
        Group.__init__(self, self, _Object(self, root_addr), "/")

    def _node(self, addr, name):
        if addr not in self._cache:
            obj = _Object(self, addr)
            self._cache[addr] = Dataset(self, obj, name) if obj.find(0x08) else Group(self, obj, name)
        return self._cache[addr]

    def _global_heap_object(self, addr, index):
        if addr not in self._gheaps:
            buf = self.buf
            if buf[addr:addr + 4] != b"GCOL":
                raise H5Error("bad global heap collection")
            size = _u(buf, addr + 8, 8)
            objs = {}
            p = addr + 16
            while p + 16 <= addr + size:
                idx, osize = _u(buf, p, 2), _u(buf, p + 8, 8)
                if idx == 0:
                    break
                objs[idx] = bytes(buf[p + 16:p + 16 + osize])
                p += 16 + (osize + 7) // 8 * 8
            self._gheaps[addr] = objs
        return self._gheaps[addr][index]

    def close(self):
        try:
            self.buf.close()
        except (BufferError, ValueError):
            pass  # a view is still alive; the mapping goes with it
        self._fh.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


# ----------------------------------------------------------------------------------------------------------------
# writing
# ----------------------------------------------------------------------------------------------------------------

def _pad8(b):
    return b + bytes(-len(b) % 8)


def _dtype_msg(dt):
    dt = np.dtype(dt)
    if dt.kind in "iu":
        bits0 = 0x08 if dt.kind == "i" else 0
        return struct.pack("<BBBBIHH", 0x10 | 0, bits0, 0, 0, dt.itemsize, 0, 8 * dt.itemsize)
    if dt.kind == "f":
        if dt.itemsize == 4:
            return struct.pack("<BBBBIHHBBBBI", 0x10 | 1, 0x20, 31, 0, 4, 0, 32, 23, 8, 0, 23, 127)
        if dt.itemsize == 8:
            return struct.pack("<BBBBIHHBBBBI", 0x10 | 1, 0x20, 63, 0, 8, 0, 64, 52, 11, 0, 52, 1023)
    if dt.kind == "S":
        return struct.pack("<BBBBI", 0x10 | 3, 0x00, 0, 0, dt.itemsize)  # null-terminated ASCII
    raise H5Error(f"cannot write dtype {dt}")


def _dataspace_msg(shape):
    rank = len(shape)
    dims = b"".join(struct.pack("<Q", s) for s in shape)
    return struct.pack("<BBB5x", 1, rank, 1 if rank else 0) + dims + dims  # current sizes, then maximum sizes


def _message(mtype, body, flags=0):
    body = _pad8(body)
    return struct.pack("<HHB3x", mtype, len(body), flags) + body


_VLEN_STR_TYPE = bytes.fromhex("19010100" "10000000" "10000000" "01000000" "00000800")  # as h5py writes `str`


class _Writer:
    def __init__(self, leaf_k):
        self.buf = bytearray()
        self.leaf_k = leaf_k
        self.gcol = None  # [address, bytes used, objects] of the open global heap collection

    def heap_string(self, raw):
        """Store one variable-length string in a global heap collection -> its 16-byte reference."""
        need = 16 + (len(raw) + 7) // 8 * 8
        if need > 4096 - 32:
            raise H5Error("string attribute too long for this writer")
        if self.gcol is None or self.gcol[1] + need + 16 > 4096:
            self.gcol = [self.alloc(bytes(4096)), 16, 0]
        addr, used, count = self.gcol
        count += 1
        obj = struct.pack("<HH4xQ", count, 0, len(raw)) + _pad8(raw)
        self.buf[addr + used:addr + used + len(obj)] = obj
        used += len(obj)
        self.buf[addr:addr + 16] = b"GCOL" + struct.pack("<B3xQ", 1, 4096)
        self.buf[addr + used:addr + used + 16] = struct.pack("<HH4xQ", 0, 0, 4096 - used)  # the free remainder
        self.gcol = [addr, used, count]
        return struct.pack("<IQI", len(raw), addr, count)

    def attr_msg(self, name, value):
        if isinstance(value, (str, bytes)):
            raw = value.encode() if isinstance(value, str) else value
            tmsg, shape, data = _VLEN_STR_TYPE, (), self.heap_string(raw)
        else:
            arr = np.asarray(value)
            if arr.dtype.kind == "b":
                arr = arr.astype(np.int8)
            if arr.dtype.kind == "U":
                arr = arr.astype("S")
            arr = np.asarray(arr.astype(arr.dtype.newbyteorder("<")), order="C")
            tmsg, shape, data = _dtype_msg(arr.dtype), arr.shape, arr.tobytes()
        nm = name.encode() + b"\0"
        smsg = _dataspace_msg(shape)
        body = struct.pack("<BBHHH", 1, 0, len(nm), len(tmsg), len(smsg)) + _pad8(nm) + _pad8(tmsg) + _pad8(smsg)
        return _message(0x0C, body + data)

    def alloc(self, data):
        self.buf += bytes(-len(self.buf) % 8)
        addr = len(self.buf)
        self.buf += data
        return addr

    def object_header(self, msgs):
        body = b"".join(msgs)
        head = struct.pack("<BBHII4x", 1, 0, len(msgs), 1, len(body))
        return self.alloc(head + body)

    def dataset(self, arr, attrs):
        arr = np.asarray(arr)
        if arr.dtype.kind == "U":
            arr = arr.astype("S")
        if arr.dtype.kind == "b":
            arr = arr.astype(np.int8)
        arr = np.asarray(arr.astype(arr.dtype.newbyteorder("<")), order="C")
        data = arr.tobytes()
        daddr = self.alloc(data) if data else UNDEF
        msgs = [_message(0x01, _dataspace_msg(arr.shape)),
                _message(0x03, _dtype_msg(arr.dtype), flags=1),
                _message(0x05, struct.pack("<BBBBI", 2, 2, 2, 1, 0)),  # fill value: late, if set, default
                _message(0x08, struct.pack("<BBQQ", 3, 1, daddr, len(data)))]
        msgs += [self.attr_msg(k, v) for k, v in attrs.items()]
        return self.object_header(msgs)

    def group(self, members, attrs):
        """members: {name: ("group", sub_members, sub_attrs) | ("dataset", array, attrs)} -> (header, btree, heap)."""
        names = sorted(members, key=lambda s: s.encode())
        if len(names) > 2 * self.leaf_k:
            raise H5Error(f"a group holds at most {2 * self.leaf_k} members in this writer")
        entries = []
        heap = bytearray(8)  # offset 0: the empty name
        for name in names:
            kind, payload, a = members[name]
            noff = len(heap)
            heap += _pad8(name.encode() + b"\0")
            if kind == "group":
                oaddr, bt, hp = self.group(payload, a)
                scratch = struct.pack("<QQ", bt, hp)
                ctype = 1
            else:
                oaddr = self.dataset(payload, a)
                scratch = bytes(16)
                ctype = 0
            entries.append((noff, struct.pack("<QQII", noff, oaddr, ctype, 0) + scratch))
        heap_size = max(len(heap) + 16, 88)
        free_off = len(heap)
        heap += struct.pack("<QQ", 1, heap_size - free_off)  # one free block: next = 1 (none), its size
        heap += bytes(heap_size - len(heap))
        hdata = self.alloc(bytes(heap))
        haddr = self.alloc(b"HEAP" + struct.pack("<B3xQQQ", 0, heap_size, free_off, hdata))
        snod = b"SNOD" + struct.pack("<BBH", 1, 0, len(entries)) + b"".join(e for _, e in entries)
        snod += bytes(8 + 40 * 2 * self.leaf_k - len(snod))
        if entries:
            saddr = self.alloc(snod)
            tree = b"TREE" + struct.pack("<BBHQQ", 0, 0, 1, UNDEF, UNDEF) + struct.pack("<QQQ", 0, saddr,
                                                                                         entries[-1][0])
        else:
            tree = b"TREE" + struct.pack("<BBHQQ", 0, 0, 0, UNDEF, UNDEF)
        tree += bytes(24 + (2 * 16 + 1) * 8 + 2 * 16 * 8 - len(tree))  # room for 2K keys + children (internal K = 16)
        baddr = self.alloc(tree)
        msgs = [_message(0x11, struct.pack("<QQ", baddr, haddr))] + [self.attr_msg(k, v) for k, v in attrs.items()]
        return self.object_header(msgs), baddr, haddr


def write(path, tree, attrs=None, leaf_k=32):
    """Write a whole file from a nested dict.

    tree: {name: numpy array | (numpy array, {attr: value}) | dict (a sub-group; its "__attrs__" key, if present,
    holds the group's attributes)}.
    """
    def convert(d):
        members, a = {}, {}
        for k, v in d.items():
            if k == "__attrs__":
                a = dict(v)
            elif isinstance(v, dict):
                sub, sa = convert(v)
                members[k] = ("group", sub, sa)
            elif isinstance(v, tuple):
                members[k] = ("dataset", v[0], dict(v[1]))
            else:
                members[k] = ("dataset", v, {})
        return members, a

    members, root_attrs = convert(tree)
    root_attrs.update(attrs or {})
    w = _Writer(leaf_k)
    w.buf += bytes(96)  # superblock, filled in last
    root, bt, hp = w.group(members, root_attrs)
    eof = len(w.buf)
    sb = SIGNATURE + struct.pack("<BBBBBBBBHHI", 0, 0, 0, 0, 0, 8, 8, 0, leaf_k, 16, 0)
    sb += struct.pack("<QQQQ", 0, UNDEF, eof, UNDEF)
    sb += struct.pack("<QQII", 0, root, 1, 0) + struct.pack("<QQ", bt, hp)
    assert len(sb) == 96
    w.buf[:96] = sb
    with open(path, "wb") as fh:
        fh.write(w.buf)
