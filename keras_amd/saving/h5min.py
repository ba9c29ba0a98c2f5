"""The subset of HDF5 that Keras weight files use, read and written without `h5py`.

`H5IOStore` (keras/src/saving/saving_lib.py:1289-1483) keeps every variable as a plain
dataset `<inner_path>/vars/<idx>` made by `group[key] = ndarray` and tags groups and bfloat16
datasets with string attributes.  h5py's defaults put that on disk in the oldest HDF5 layout:
superblock version 0, version-1 object headers, groups as symbol tables (a version-1 B-tree
of symbol-table nodes plus a local heap of names), contiguous little-endian datasets,
version-1 attribute messages whose strings are variable-length entries of a global heap.
This module reads and writes exactly that (HDF5 File Format Specification, version 1.1):
no chunking, no compression, no new-style (link-message) groups.  It executes nothing from
a file; anything outside the subset raises `H5FormatError`.

`load(data) -> Group`, `dump(group) -> bytes`.
"""

import struct

import numpy as np

SIGNATURE = b"\x89HDF\r\n\x1a\n"
UNDEF = 0xFFFFFFFFFFFFFFFF
LEAF_K = 4      # symbol-table nodes hold up to 2 * LEAF_K entries
INTERNAL_K = 16  # B-tree nodes hold up to 2 * INTERNAL_K children
BTREE_NODE_BYTES = 24 + (2 * INTERNAL_K + 1) * 8 + 2 * INTERNAL_K * 8
SNOD_BYTES = 8 + 2 * LEAF_K * 40

MSG_NIL, MSG_DATASPACE, MSG_DATATYPE, MSG_FILL, MSG_LAYOUT = 0x0, 0x1, 0x3, 0x5, 0x8
MSG_ATTRIBUTE, MSG_CONTINUATION, MSG_SYMBOL_TABLE = 0xC, 0x10, 0x11


class H5FormatError(ValueError):
    pass


class Dataset:
    """An array and its attributes.  Arrays of numpy void dtype (`V2`: how bfloat16 bit
    patterns travel) are stored as opaque elements."""

    def __init__(self, value, attrs=None):
        self.value = value
        self.attrs = dict(attrs or {})


class Group(dict):
    """Children by name (Group or Dataset) and attributes."""

    def __init__(self, *args, attrs=None, **kwargs):
        super().__init__(*args, **kwargs)
        self.attrs = dict(attrs or {})

    def lookup(self, path):
        """Object at a '/'-separated path, or None."""
        node = self
        for part in [p for p in path.split("/") if p]:
            if not isinstance(node, Group) or part not in node:
                return None
            node = node[part]
        return node

    def require_group(self, path):
        node = self
        for part in [p for p in path.split("/") if p]:
            nxt = node.get(part)
            if nxt is None:
                nxt = node[part] = Group()
            elif not isinstance(nxt, Group):
                raise H5FormatError(f"'{part}' in '{path}' is a dataset, not a group")
            node = nxt
        return node


def _pad8(n):
    return (n + 7) & ~7


# --------------------------------------------------------------------------- reading


class _Reader:
    def __init__(self, data):
        self.d = bytes(data)
        self.gcol = {}

    def fail(self, what):
        raise H5FormatError(f"unsupported or malformed HDF5 content: {what}")

    def u(self, fmt, off):
        try:
            return struct.unpack_from("<" + fmt, self.d, off)
        except struct.error:
            self.fail(f"read past the end of the file at {off}")

    def root(self):
        d = self.d
        if d[:8] != SIGNATURE:
            self.fail("no HDF5 signature at offset 0")
        if d[8] != 0:
            self.fail(f"superblock version {d[8]} (only version 0 is read)")
        if d[13] != 8 or d[14] != 8:
            self.fail("offsets / lengths that are not 8 bytes wide")
        (base,) = self.u("Q", 24)
        if base != 0:
            self.fail("a non-zero base address")
        _, ohdr = self.u("QQ", 56)
        return self.read_object(ohdr, depth=0)

    def messages(self, addr):
        ver, _, nmsg, _, hsize = self.u("BBHII", addr)
        if ver != 1:
            self.fail(f"object header version {ver} at {addr}")
        blocks = [(addr + 16, addr + 16 + hsize)]
        out = []
        while blocks and len(out) < nmsg:
            p, end = blocks.pop(0)
            while p + 8 <= end and len(out) < nmsg:
                mtype, size, _ = self.u("HHB", p)
                body = p + 8
                if body + size > len(self.d):
                    self.fail("a header message that runs past the end of the file")
                out.append((mtype, body, size))
                if mtype == MSG_CONTINUATION:
                    caddr, clen = self.u("QQ", body)
                    blocks.append((caddr, caddr + clen))
                p = body + size
        return out

    def read_object(self, addr, depth):
        if depth > 64:
            self.fail("groups nested deeper than 64 levels")
        msgs = self.messages(addr)
        kinds = {m[0] for m in msgs}
        attrs = {}
        for mtype, body, size in msgs:
            if mtype == MSG_ATTRIBUTE:
                name, value = self.attribute(body, size)
                attrs[name] = value
        if MSG_SYMBOL_TABLE in kinds:
            body = next(b for t, b, _ in msgs if t == MSG_SYMBOL_TABLE)
            btree, heap = self.u("QQ", body)
            group = Group(attrs=attrs)
            for name, child in self.symbols(btree, heap, 0):
                group[name] = self.read_object(child, depth + 1)
            return group
        if MSG_LAYOUT in kinds:
            space = next(((b, s) for t, b, s in msgs if t == MSG_DATASPACE), None)
            dtype = next(((b, s) for t, b, s in msgs if t == MSG_DATATYPE), None)
            layout = next((b for t, b, _ in msgs if t == MSG_LAYOUT))
            if space is None or dtype is None:
                self.fail(f"dataset at {addr} without dataspace or datatype")
            shape = self.dataspace(space[0])
            np_dtype, kind = self.datatype(dtype[0])
            if kind == "vlen_str":
                self.fail("variable-length string datasets")
            raw = self.layout_bytes(layout, int(np.prod(shape, dtype=np.int64)) * np_dtype.itemsize)
            value = np.frombuffer(raw, dtype=np_dtype).reshape(shape).copy()
            return Dataset(value, attrs)
        self.fail(f"object at {addr} is neither an old-style group nor a dataset "
                  f"(message types {sorted(kinds)})")

    def symbols(self, btree, heap, depth):
        if self.d[heap:heap + 4] != b"HEAP":
            self.fail(f"no local heap at {heap}")
        (names,) = self.u("Q", heap + 24)
        if depth > 8 or self.d[btree:btree + 4] != b"TREE":
            self.fail(f"no B-tree node at {btree}")
        ntype, level, used = self.u("BBH", btree + 4)
        if ntype != 0:
            self.fail("a chunk B-tree where a group B-tree belongs")
        p = btree + 24
        for _ in range(used):
            _, child = self.u("QQ", p)
            p += 16
            if level > 0:
                yield from self.symbols(child, heap, depth + 1)
                continue
            if self.d[child:child + 4] != b"SNOD":
                self.fail(f"no symbol-table node at {child}")
            (count,) = self.u("H", child + 6)
            q = child + 8
            for _ in range(count):
                name_off, ohdr = self.u("QQ", q)
                q += 40
                start = names + name_off
                end = self.d.find(b"\0", start)
                if end < 0:
                    self.fail("an unterminated link name")
                yield self.d[start:end].decode("utf-8"), ohdr

    def dataspace(self, body):
        ver, rank, flags = self.u("BBB", body)
        if ver == 1:
            p = body + 8
        elif ver == 2:
            (stype,) = self.u("B", body + 3)
            if stype == 2:
                self.fail("a null dataspace")
            p = body + 4
        else:
            self.fail(f"dataspace version {ver}")
        return tuple(self.u("Q" * rank, p)) if rank else ()

    def datatype(self, body):
        """-> (numpy dtype of one element, kind) with kind in
        'number' | 'opaque' | 'string' | 'vlen_str'."""
        cv, b0, b1, _, size = self.u("BBBBI", body)
        cls = cv & 0x0F
        if cls in (0, 1) and (b0 & 1):
            self.fail("big-endian numbers")
        if cls == 0:
            signed = bool(b0 & 0x08)
            if size not in (1, 2, 4, 8):
                self.fail(f"{size}-byte integers")
            return np.dtype(("<i" if signed else "<u") + str(size)), "number"
        if cls == 1:
            _, precision, _, exp_bits, _, man_bits, _ = self.u("HHBBBBI", body + 8)
            known = {(2, 5, 10): "<f2", (4, 8, 23): "<f4", (8, 11, 52): "<f8"}
            if (size, exp_bits, man_bits) not in known or precision != 8 * size:
                self.fail(f"a float type of {size} bytes with {exp_bits}+{man_bits} bits")
            return np.dtype(known[(size, exp_bits, man_bits)]), "number"
        if cls == 3:
            return np.dtype(f"S{size}"), "string"
        if cls == 5:
            return np.dtype(f"V{size}"), "opaque"
        if cls == 9:
            if (b0 & 0x0F) != 1:
                self.fail("variable-length sequences")
            return np.dtype("V16"), "vlen_str"
        self.fail(f"datatype class {cls}")

    def datatype_bytes(self, body):
        """Length of the datatype message starting at `body` (needed inside attributes)."""
        cv, b0, _, _, _ = self.u("BBBBI", body)
        cls = cv & 0x0F
        if cls == 0:
            return 12
        if cls == 1:
            return 20
        if cls == 3:
            return 8
        if cls == 5:
            return 8 + _pad8(b0)
        if cls == 9:
            return 8 + self.datatype_bytes(body + 8)
        self.fail(f"datatype class {cls}")

    def layout_bytes(self, body, nbytes):
        ver, cls = self.u("BB", body)
        if ver != 3:
            self.fail(f"data layout version {ver}")
        if cls == 0:
            (size,) = self.u("H", body + 2)
            raw = self.d[body + 4:body + 4 + size]
        elif cls == 1:
            addr, size = self.u("QQ", body + 2)
            if nbytes == 0:
                return b""
            if addr == UNDEF:
                self.fail("a dataset whose storage was never allocated")
            raw = self.d[addr:addr + size]
        else:
            self.fail("chunked datasets")
        if len(raw) < nbytes:
            self.fail("a dataset shorter than its shape says")
        return raw[:nbytes]

    def vlen_string(self, raw):
        length, addr, index = struct.unpack("<IQI", raw)
        if length == 0:
            return ""
        if addr not in self.gcol:
            if self.d[addr:addr + 4] != b"GCOL":
                self.fail(f"no global heap collection at {addr}")
            (total,) = self.u("Q", addr + 8)
            objs, p = {}, addr + 16
            while p + 16 <= addr + total:
                idx, _, _, size = self.u("HHIQ", p)
                if idx == 0:
                    break
                objs[idx] = self.d[p + 16:p + 16 + size]
                p += 16 + _pad8(size)
            self.gcol[addr] = objs
        if index not in self.gcol[addr]:
            self.fail("a global-heap reference to a missing object")
        return self.gcol[addr][index][:length].decode("utf-8")

    def attribute(self, body, size):
        ver, _, name_len, dt_len, ds_len = self.u("BBHHH", body)
        p = body + 8
        if ver == 3:
            p += 1  # name character set
        if ver not in (1, 2, 3):
            self.fail(f"attribute message version {ver}")
        step = _pad8 if ver == 1 else (lambda n: n)
        name = self.d[p:p + name_len].split(b"\0")[0].decode("utf-8")
        p += step(name_len)
        dt_at = p
        p += step(dt_len)
        ds_at = p
        p += step(ds_len)
        shape = self.dataspace(ds_at)
        np_dtype, kind = self.datatype(dt_at)
        count = int(np.prod(shape, dtype=np.int64))
        raw = self.d[p:p + count * np_dtype.itemsize]
        if kind == "vlen_str":
            items = [self.vlen_string(raw[16 * i:16 * i + 16]) for i in range(count)]
            value = items[0] if shape == () else np.array(items, dtype=object).reshape(shape)
        elif kind == "string":
            items = [bytes(x).split(b"\0")[0].decode("utf-8") for x in np.frombuffer(raw, dtype=np_dtype)]
            value = items[0] if shape == () else np.array(items, dtype=object).reshape(shape)
        else:
            arr = np.frombuffer(raw, dtype=np_dtype).reshape(shape).copy()
            value = arr[()] if shape == () else arr
        return name, value


def load(data):
    """Parse the bytes of an HDF5 file of the subset described above into a `Group` tree."""
    return _Reader(data).root()


# --------------------------------------------------------------------------- writing


def _datatype_message(dtype):
    """Datatype message body for a numpy dtype, as h5py writes it."""
    dtype = np.dtype(dtype)
    if dtype.kind in "iu":
        bits = 0x08 if dtype.kind == "i" else 0x00
        return struct.pack("<BBBBIHH", 0x10, bits, 0, 0, dtype.itemsize, 0, 8 * dtype.itemsize)
    if dtype.kind == "b":  # numpy bool: h5py stores an enum; the plain byte is enough here
        return struct.pack("<BBBBIHH", 0x10, 0x00, 0, 0, 1, 0, 8)
    if dtype.kind == "f":
        exp_bits, man_bits, bias = {2: (5, 10, 15), 4: (8, 23, 127), 8: (11, 52, 1023)}[dtype.itemsize]
        sign_pos = 8 * dtype.itemsize - 1
        return struct.pack("<BBBBIHHBBBBI", 0x11, 0x20, sign_pos, 0, dtype.itemsize, 0,
                           8 * dtype.itemsize, man_bits, exp_bits, 0, man_bits, bias)
    if dtype.kind == "V":  # opaque bytes with an empty tag
        return struct.pack("<BBBBI", 0x15, 0, 0, 0, dtype.itemsize)
    raise H5FormatError(f"arrays of dtype {dtype} cannot be written")


_VLEN_STR_TYPE = struct.pack("<BBBBI", 0x19, 0x01, 0x01, 0, 16) + struct.pack("<BBBBIHH", 0x10, 0, 0, 0, 1, 0, 8)


def _dataspace_message(shape, with_max):
    rank = len(shape)
    body = struct.pack("<BBBBI", 1, rank, 1 if (with_max and rank) else 0, 0, 0)
    body += struct.pack("<" + "Q" * rank, *shape)
    if with_max and rank:
        body += struct.pack("<" + "Q" * rank, *shape)
    return body


class _Writer:
    def __init__(self):
        self.buf = bytearray()
        self.strings = []  # global-heap objects (index = position + 1)

    def alloc(self, nbytes):
        addr = len(self.buf)
        self.buf += b"\0" * _pad8(nbytes)
        return addr

    def put(self, addr, data):
        self.buf[addr:addr + len(data)] = data

    # -- attributes -------------------------------------------------------------------
    def attribute_message(self, name, value, gcol_addr):
        nm = name.encode("utf-8") + b"\0"
        if isinstance(value, str):
            self.strings.append(value.encode("utf-8"))
            dt, ds = _VLEN_STR_TYPE, _dataspace_message((), False)
            data = struct.pack("<IQI", len(self.strings[-1]), gcol_addr, len(self.strings))
        else:
            arr = np.asarray(value)
            if arr.dtype.kind not in "iufb":
                raise H5FormatError(f"attribute '{name}' of type {arr.dtype} cannot be written")
            dt, ds = _datatype_message(arr.dtype), _dataspace_message(arr.shape, False)
            data = arr.astype(arr.dtype.newbyteorder("<")).tobytes()
        body = struct.pack("<BBHHH", 1, 0, len(nm), len(dt), len(ds))
        for part in (nm, dt, ds):
            body += part + b"\0" * (_pad8(len(part)) - len(part))
        body += data
        return MSG_ATTRIBUTE, body

    def object_header(self, messages):
        """Version-1 object header holding `messages` [(type, body, flags)] in one block."""
        blob = bytearray()
        for mtype, body, flags in messages:
            size = _pad8(len(body))
            blob += struct.pack("<HHBBBB", mtype, size, flags, 0, 0, 0) + body + b"\0" * (size - len(body))
        addr = self.alloc(16 + len(blob))
        self.put(addr, struct.pack("<BBHII", 1, 0, len(messages), 1, len(blob)) + b"\0" * 4 + bytes(blob))
        return addr

    # -- objects ------------------------------------------------------------------------
    def write_dataset(self, ds, gcol_addr):
        arr = np.asarray(ds.value)  # tobytes() below emits C order whatever the strides
        if arr.dtype.kind in "iuf" and arr.dtype.byteorder == ">":
            arr = arr.astype(arr.dtype.newbyteorder("<"))
        raw = arr.tobytes()
        data_addr = UNDEF
        if raw:
            data_addr = self.alloc(len(raw))
            self.put(data_addr, raw)
        msgs = [
            (MSG_DATASPACE, _dataspace_message(arr.shape, True), 0),
            (MSG_DATATYPE, _datatype_message(arr.dtype), 1),
            (MSG_FILL, struct.pack("<BBBB", 2, 2, 2, 1) + struct.pack("<I", 0), 1),
            (MSG_LAYOUT, struct.pack("<BBQQ", 3, 1, data_addr, len(raw)), 0),
        ]
        for name, value in ds.attrs.items():
            mtype, body = self.attribute_message(name, value, gcol_addr)
            msgs.append((mtype, body, 0))
        return self.object_header(msgs)

    def write_group(self, group, gcol_addr):
        """-> (object header address, B-tree address, local heap address)."""
        children = []
        for name in sorted(group, key=lambda n: n.encode("utf-8")):
            child = group[name]
            if isinstance(child, Group):
                children.append((name, self.write_group(child, gcol_addr)[0]))
            elif isinstance(child, Dataset):
                children.append((name, self.write_dataset(child, gcol_addr)))
            else:
                raise H5FormatError(f"'{name}' is neither a Group nor a Dataset")
        # local heap: the empty name at offset 0, then the names, then one free block
        names = bytearray(b"\0" * 8)
        offsets = []
        for name, _ in children:
            offsets.append(len(names))
            enc = name.encode("utf-8") + b"\0"
            names += enc + b"\0" * (_pad8(len(enc)) - len(enc))
        free_at = len(names)
        free_len = max(16, 88 - free_at)
        names += struct.pack("<QQ", 1, free_len) + b"\0" * (free_len - 16)
        heap = self.alloc(32 + len(names))
        self.put(heap, b"HEAP" + struct.pack("<BBBBQQQ", 0, 0, 0, 0, len(names), free_at, heap + 32) + bytes(names))
        # symbol-table nodes of at most 2 * LEAF_K entries, evenly filled
        entries = list(zip(offsets, [c[1] for c in children]))
        n_leaves = max(1, -(-len(entries) // (2 * LEAF_K)))
        leaves = []  # (address, heap offset of its last name)
        for i in range(n_leaves):
            part = entries[i * len(entries) // n_leaves:(i + 1) * len(entries) // n_leaves]
            addr = self.alloc(SNOD_BYTES)
            blob = b"SNOD" + struct.pack("<BBH", 1, 0, len(part))
            for off, ohdr in part:
                blob += struct.pack("<QQII", off, ohdr, 0, 0) + b"\0" * 16
            self.put(addr, blob)
            leaves.append((addr, part[-1][0] if part else 0))
        # B-tree over them, bottom up, nodes of at most 2 * INTERNAL_K children
        level, nodes = 0, leaves
        while True:
            n_nodes = max(1, -(-len(nodes) // (2 * INTERNAL_K)))
            addrs = [self.alloc(BTREE_NODE_BYTES) for _ in range(n_nodes)]
            parents = []
            for i, addr in enumerate(addrs):
                part = nodes[i * len(nodes) // n_nodes:(i + 1) * len(nodes) // n_nodes]
                left = addrs[i - 1] if i > 0 else UNDEF
                right = addrs[i + 1] if i + 1 < n_nodes else UNDEF
                first_key = 0 if i == 0 else parents[-1][1]
                blob = b"TREE" + struct.pack("<BBHQQ", 0, level, len(part) if entries else 0, left, right)
                blob += struct.pack("<Q", first_key)
                for child, last_key in (part if entries else []):
                    blob += struct.pack("<QQ", child, last_key)
                self.put(addr, blob)
                parents.append((addr, part[-1][1] if part else 0))
            if n_nodes == 1:
                btree = addrs[0]
                break
            level, nodes = level + 1, parents
        msgs = [(MSG_SYMBOL_TABLE, struct.pack("<QQ", btree, heap), 0)]
        for name, value in group.attrs.items():
            mtype, body = self.attribute_message(name, value, gcol_addr)
            msgs.append((mtype, body, 0))
        return self.object_header(msgs), btree, heap


def _count_string_bytes(group):
    total = sum(16 + _pad8(len(v.encode("utf-8"))) for v in group.attrs.values() if isinstance(v, str))
    for child in group.values():
        if isinstance(child, Group):
            total += _count_string_bytes(child)
        else:
            total += sum(16 + _pad8(len(v.encode("utf-8"))) for v in child.attrs.values()
                         if isinstance(v, str))
    return total


def dump(root):
    """Serialize a `Group` tree to the bytes of an HDF5 file (layout described above)."""
    if not isinstance(root, Group):
        raise H5FormatError("the root must be a Group")
    w = _Writer()
    w.alloc(96)  # superblock, written last
    # one global heap collection for every string attribute, placed first so that its
    # address is known while the attributes are written
    gcol_bytes = max(4096, _pad8(16 + _count_string_bytes(root) + 16))
    gcol = w.alloc(gcol_bytes)
    ohdr, btree, heap = w.write_group(root, gcol)
    blob = bytearray(b"GCOL" + struct.pack("<BBBBQ", 1, 0, 0, 0, gcol_bytes))
    for i, s in enumerate(w.strings):
        blob += struct.pack("<HHIQ", i + 1, 0, 0, len(s)) + s + b"\0" * (_pad8(len(s)) - len(s))
    free = gcol_bytes - len(blob)
    blob += struct.pack("<HHIQ", 0, 0, 0, free)  # object 0: the free space (size includes its header)
    w.put(gcol, bytes(blob))
    eof = len(w.buf)
    sb = SIGNATURE + struct.pack("<BBBBBBBBHHI", 0, 0, 0, 0, 0, 8, 8, 0, LEAF_K, INTERNAL_K, 0)
    sb += struct.pack("<QQQQ", 0, UNDEF, eof, UNDEF)
    sb += struct.pack("<QQII", 0, ohdr, 1, 0) + struct.pack("<QQ", btree, heap)
    w.put(0, sb)
    return bytes(w.buf)
