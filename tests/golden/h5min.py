"""A minimal reader for the HDF5 files Keras writes for layer weights (test infrastructure).

Understands what those files use and nothing else: superblock version 0 with 8-byte offsets and
lengths, old-style groups (symbol table message -> version-1 B-tree -> symbol table nodes -> local
heap), version-1 object headers with continuation blocks, simple dataspaces, fixed-point / IEEE
little-endian datatypes and contiguous (or compact) data layout.  Nothing in the file is executed.
"""
import struct

import numpy as np

UNDEF = 0xFFFFFFFFFFFFFFFF


class H5Error(Exception):
    pass


class H5File:
    def __init__(self, path):
        self.d = open(path, 'rb').read()
        d = self.d
        if d[:8] != b'\x89HDF\r\n\x1a\n':
            raise H5Error('not an HDF5 file')
        if d[8] != 0 or d[13] != 8 or d[14] != 8:
            raise H5Error('only superblock version 0 with 8-byte offsets and lengths is understood')
        self.base = self.u64(24)
        # root group symbol table entry follows the four superblock addresses
        self.root_header = self.u64(24 + 32 + 8)

    def u16(self, o):
        return struct.unpack_from('<H', self.d, o)[0]

    def u32(self, o):
        return struct.unpack_from('<I', self.d, o)[0]

    def u64(self, o):
        return struct.unpack_from('<Q', self.d, o)[0]

    def messages(self, addr):
        """(type, payload offset, payload size) of every message of the object header at addr."""
        d, o = self.d, addr + self.base
        if d[o] != 1:
            raise H5Error('only version-1 object headers are understood')
        n_msgs, size = self.u16(o + 2), self.u32(o + 8)
        blocks = [(o + 16, size)]
        out = []
        while blocks and len(out) < n_msgs:
            p, left = blocks.pop(0)
            while left >= 8 and len(out) < n_msgs:
                mtype, msize = self.u16(p), self.u16(p + 2)
                out.append((mtype, p + 8, msize))
                if mtype == 0x0010:  # continuation: offset, length
                    blocks.append((self.u64(p + 8) + self.base, self.u64(p + 16)))
                p += 8 + msize
                left -= 8 + msize
        return out

    def heap_name(self, heap_addr, off):
        h = heap_addr + self.base
        if self.d[h:h + 4] != b'HEAP':
            raise H5Error('bad local heap')
        data = self.u64(h + 24) + self.base
        end = self.d.index(b'\x00', data + off)
        return self.d[data + off:end].decode()

    def group_entries(self, btree_addr, heap_addr):
        """(name, object header address) of the links below a version-1 group B-tree."""
        t = btree_addr + self.base
        if self.d[t:t + 4] != b'TREE' or self.d[t + 4] != 0:
            raise H5Error('bad group B-tree node')
        level, used = self.d[t + 5], self.u16(t + 6)
        out = []
        p = t + 24  # keys and children alternate, starting with key 0
        for i in range(used):
            child = self.u64(p + 8 + 16 * i)
            if level > 0:
                out += self.group_entries(child, heap_addr)
                continue
            s = child + self.base
            if self.d[s:s + 4] != b'SNOD':
                raise H5Error('bad symbol table node')
            for k in range(self.u16(s + 6)):
                e = s + 8 + 40 * k
                out.append((self.heap_name(heap_addr, self.u64(e)), self.u64(e + 8)))
        return out

    def datasets(self, addr=None, prefix=''):
        """{path: numpy array} of every dataset below the group at addr (default: the root group)."""
        addr = self.root_header if addr is None else addr
        msgs = self.messages(addr)
        out = {}
        for mtype, p, _ in msgs:
            if mtype == 0x0011:  # symbol table: this object is a group
                for name, child in self.group_entries(self.u64(p), self.u64(p + 8)):
                    out.update(self.datasets(child, prefix + '/' + name))
                return out
        shape = dtype = data = None
        for mtype, p, size in msgs:
            if mtype == 0x0001:  # dataspace
                ver, rank, flags = self.d[p], self.d[p + 1], self.d[p + 2]
                dims = p + (8 if ver == 1 else 4)
                shape = tuple(self.u64(dims + 8 * i) for i in range(rank))
            elif mtype == 0x0003:  # datatype
                cls, bits0, nbytes = self.d[p] & 15, self.d[p + 1], self.u32(p + 4)
                if bits0 & 1:
                    raise H5Error('big-endian data')
                if cls == 1:
                    dtype = {2: '<f2', 4: '<f4', 8: '<f8'}[nbytes]
                elif cls == 0:
                    dtype = ('<i' if bits0 & 8 else '<u') + str(nbytes)
            elif mtype == 0x0008:  # data layout
                ver, cls = self.d[p], self.d[p + 1]
                if ver != 3:
                    raise H5Error('only version-3 layout messages are understood')
                if cls == 1:
                    a, n = self.u64(p + 2), self.u64(p + 10)
                    data = None if a == UNDEF else self.d[a + self.base:a + self.base + n]
                elif cls == 0:
                    n = self.u16(p + 2)
                    data = self.d[p + 4:p + 4 + n]
                else:
                    raise H5Error('chunked datasets are not understood')
        if shape is not None and dtype is not None and data is not None:
            out[prefix] = np.frombuffer(data, dtype=dtype).reshape(shape).copy()
        return out
