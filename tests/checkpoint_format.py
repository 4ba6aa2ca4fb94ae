"""An independent reader / writer of the reference's table-file layout (common/serialize.h,
checkpoint/checkpoint.cc:444-509), written with `struct`: the second reading of the format that
the library's C++ reader and writer are checked against, itself pinned against files written by
the reference's own serializer (tests/golden/ref_*.sparse, ref_*.dense)."""
import struct

import numpy as np


class Cursor:
    def __init__(self, data):
        self.d, self.at = data, 0

    def take(self, fmt):
        v = struct.unpack_from("<" + fmt, self.d, self.at)
        self.at += struct.calcsize("<" + fmt)
        return v[0] if len(v) == 1 else v

    def string(self):                      # serialize.h:86-94
        n = self.take("Q")
        s = self.d[self.at:self.at + n].decode()
        self.at += n
        return s

    def tensor(self):                      # serialize.h:156-176
        assert self.take("B") == 0         # Layout::kStride
        rank = self.take("Q")
        dims = [self.take("q") for _ in range(rank)]
        assert self.take("B") == 11        # DType::kFloat32
        n = int(np.prod(dims)) if dims else 1
        v = np.frombuffer(self.d, np.float32, n, self.at).copy()
        self.at += 4 * n
        return dims, v

    def value(self):                       # serialize.h:296-298, 242-272
        dims, val = self.tensor()
        states = {}
        for _ in range(self.take("Q")):
            st = self.take("I")
            states[st] = self.tensor()[1]
        counters = {}
        for _ in range(self.take("Q")):
            st = self.take("I")
            counters[st] = self.take("q")
        return dims, val, states, counters


def parse_sparse(path):
    c = Cursor(open(path, "rb").read())
    head = dict(type=c.take("B"), id=c.take("Q"), name=c.string(), dim=c.take("q"), dtype=c.take("B"),
                init=c.take("B"))
    head["conf"] = {c.string(): c.string() for _ in range(c.take("Q"))}
    slots = []
    for _ in range(c.take("Q")):
        rows = []
        for _ in range(c.take("Q")):
            key = c.take("Q")
            rows.append((key,) + c.value())
        slots.append(rows)
    assert c.at == len(c.d)
    return head, slots


def pack_tensor(v, dims=None):
    v = np.ascontiguousarray(v, np.float32)
    dims = list(dims) if dims is not None else [v.size]
    return struct.pack("<BQ", 0, len(dims)) + b"".join(struct.pack("<q", d) for d in dims) + b"\x0b" + v.tobytes()


def pack_string(s):
    return struct.pack("<Q", len(s)) + s.encode()


def pack_value(val, states, counters, dims=None):
    out = pack_tensor(val, dims) + struct.pack("<Q", len(states))
    for st, v in states.items():
        out += struct.pack("<I", st) + pack_tensor(v, dims)
    out += struct.pack("<Q", len(counters))
    for st, c in counters.items():
        out += struct.pack("<Iq", st, c)
    return out


def parse_dense(path):
    c = Cursor(open(path, "rb").read())
    head = dict(type=c.take("B"), id=c.take("Q"), name=c.string())
    dims, val, states, counters = c.value()
    assert c.at == len(c.d)
    return head, dims, val, states, counters


def pack_rows(rows):
    """std::vector<Tensor> of 1-D fp32 rows (serialize.h:214-228): what a pull reply carries."""
    rows = np.ascontiguousarray(rows, np.float32)
    return struct.pack("<Q", rows.shape[0]) + b"".join(pack_tensor(r) for r in rows)


def parse_rows(data):
    c = Cursor(bytes(data))
    out = []
    for _ in range(c.take("Q")):
        dims, v = c.tensor()
        assert len(dims) == 1
        out.append(v)
    assert c.at == len(c.d)
    return np.array(out, np.float32).reshape(len(out), -1)

