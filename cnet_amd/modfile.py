"""Reader and writer of upstream CNet's .mod model files (impl/model_saver.h:483-967 upstream) for Python callers of
the C ABI: the stream is a big-endian int32 magic number followed by one record per function,

    type id, uid, input length, output size, number of producers, producer uids,
    CInput: re[len], im[len] | CEmbedding: dim, slots, vocab, re[len], im[len] | Linear: in1, in2

with every int32 / float32 big-endian.  `loads` returns the records as dicts (parameters as float32 arrays), `dumps`
writes the same bytes back.  The C++ facade has the same as ModelSaver (cnet_amd/host/model_saver.hpp).
"""
import struct

import numpy as np

MAGIC = 0xABCDE0EE
# type ids of impl/cnet.h:31-44
HADAMARD, EMBEDDING, LINEAR, FOURIER, CROSS_ENTROPY, RESIDUAL, SOFTMAX, INPUT, CRELU, GELU, L2OUT, TRIANG_FOURIER = range(1, 13)
_KNOWN = set(range(1, 13))


def loads(blob):
    pos = 0

    def i32(count=1):
        nonlocal pos
        if pos + 4 * count > len(blob):
            raise ValueError("truncated .mod stream at byte %d" % pos)
        vals = struct.unpack_from(">%di" % count, blob, pos)
        pos += 4 * count
        return vals

    def f32(count):
        nonlocal pos
        if count < 0 or pos + 4 * count > len(blob):
            raise ValueError("truncated parameter block at byte %d" % pos)
        arr = np.frombuffer(blob, ">f4", count, pos).astype(np.float32)
        pos += 4 * count
        return arr

    if len(blob) < 4 or struct.unpack_from(">I", blob, 0)[0] != MAGIC:
        raise ValueError("not a CNet model (magic number)")
    pos = 4
    recs = []
    while pos < len(blob):
        kind, uid, in_len, out_size, nprev = i32(5)
        if kind not in _KNOWN:
            raise ValueError("cannot restore layer of ID %d" % kind)
        if nprev < 0 or in_len < 0:
            raise ValueError("corrupt record for uid %d" % uid)
        rec = dict(type=kind, uid=uid, in_len=in_len, out_size=out_size, prev=list(i32(nprev)) if nprev else [])
        if kind == EMBEDDING:
            rec["dim"], rec["slots"], rec["vocab"] = i32(3)
        if kind in (INPUT, EMBEDDING):
            rec["re"] = f32(in_len)
            rec["im"] = f32(in_len)
        if kind == LINEAR:
            rec["in1"], rec["in2"] = i32(2)
        recs.append(rec)
    return recs


def dumps(recs):
    out = [struct.pack(">I", MAGIC)]
    for r in recs:
        out.append(struct.pack(">5i", r["type"], r["uid"], r["in_len"], r["out_size"], len(r["prev"])))
        if r["prev"]:
            out.append(struct.pack(">%di" % len(r["prev"]), *r["prev"]))
        if r["type"] == EMBEDDING:
            out.append(struct.pack(">3i", r["dim"], r["slots"], r["vocab"]))
        if r["type"] in (INPUT, EMBEDDING):
            for plane in (r["re"], r["im"]):
                a = np.ascontiguousarray(plane, np.float32)
                if a.shape != (r["in_len"],):
                    raise ValueError("uid %d: parameter plane has %r values, record says %d" % (r["uid"], a.shape, r["in_len"]))
                out.append(a.astype(">f4").tobytes())
        if r["type"] == LINEAR:
            out.append(struct.pack(">2i", r["in1"], r["in2"]))
    return b"".join(out)


def load(path):
    with open(path, "rb") as f:
        return loads(f.read())


def save(path, recs):
    with open(path, "wb") as f:
        f.write(dumps(recs))
