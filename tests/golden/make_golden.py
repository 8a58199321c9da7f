"""Writes the fixtures of this folder.  Run from the repository root:

    python tests/golden/make_golden.py

The reference holds no golden vectors, known-answer tests or fixtures for its paged KV path, and
its kernels cannot run here, so none of these files comes from the reference.  Each one states what
a published format, the reference's documented host semantics or plain mathematics fixes, computed
here with numpy and Python arithmetic only: this script imports neither the oracle nor the library,
so that both can be checked against what it writes.

  e4m3fn_table.json     the 256 values of OCP FP8 E4M3FN (bias 7, no infinities, 0x7F / 0xFF = NaN)
                        and encode cases: exact values, midpoints (ties to the even code), the
                        neighbours of midpoints, saturation at +-448
  int8_rows.json        rows quantised per (token, head): scale = fp16(absmax / 127), code =
                        clamp(round_half_even(x * fp32(1 / scale)), -127, 127) -- the precedent
                        find_absmax_kernel / quantize_to_int8_kernel, layer_int8_dual.cu:239-293,
                        with the fp16 scale the KV pages store -- including .5 ties and all-zero rows
  block_pool_trace.json a scripted alloc / free scenario on the LIFO free stack of
                        BlockPool (block_pool.cpp:18-105): ids 0, 1, 2, ... first, freed ids back
                        last-in-first-out, -1 when empty
  config1_decode.json   BASELINE config 1 (512 tokens, 4 KV heads x 128, fp16, 16 Q heads, 256
                        blocks of 16 tokens, 32 of them in a shuffled table): the attention output
                        softmax(Q K^T / sqrt(128)) V in fp64 on the fp16-rounded inputs, which
                        inputs() below regenerates from the seed (their SHA-256 is in the file)
"""
import hashlib
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


# ---- a generator that does not depend on numpy's Generator staying the same ------------
def splitmix64(n, seed):
    """n 64-bit words of the splitmix64 sequence (Steele, Lea, Flood 2014) started at `seed`."""
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + np.uint64(0x9E3779B97F4A7C15) * np.arange(1, n + 1, dtype=np.uint64))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def normals(n, seed):
    """n standard normal fp32 values: Box-Muller on pairs of 53-bit uniforms."""
    m = (n + 1) // 2
    w = splitmix64(2 * m, seed)
    u1 = ((w[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) / 2.0 ** 53        # (0, 1]
    u2 = (w[1::2] >> np.uint64(11)).astype(np.float64) / 2.0 ** 53                # [0, 1)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.stack([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)], axis=1).reshape(-1)
    return z[:n].astype(np.float32)


def fisher_yates(n, seed):
    w = splitmix64(n, seed)
    p = np.arange(n, dtype=np.int32)
    for i in range(n - 1, 0, -1):
        j = int(w[i] % np.uint64(i + 1))
        p[i], p[j] = p[j], p[i]
    return p


# ---- config 1 -----------------------------------------------------------------------
CFG1 = dict(L=1, KVH=4, QH=16, D=128, bs=16, NB=256, tokens=512, seed=1)


def config1_inputs():
    """table [32] int32, k, v [512, 4, 128] and q [16, 128] as fp16 bit patterns (uint16)"""
    c = CFG1
    table = fisher_yates(c["NB"], c["seed"])[: c["tokens"] // c["bs"]].copy()
    n = c["tokens"] * c["KVH"] * c["D"]
    k = normals(n, c["seed"] + 1).astype(np.float16).view(np.uint16).reshape(c["tokens"], c["KVH"], c["D"])
    v = normals(n, c["seed"] + 2).astype(np.float16).view(np.uint16).reshape(c["tokens"], c["KVH"], c["D"])
    q = normals(c["QH"] * c["D"], c["seed"] + 3).astype(np.float16).view(np.uint16).reshape(c["QH"], c["D"])
    return table, k, v, q


def inputs_digest(table, k, v, q):
    h = hashlib.sha256()
    for a in (table, k, v, q):
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def config1():
    c = CFG1
    table, k, v, q = config1_inputs()
    kf, vf, qf = (a.view(np.float16).astype(np.float64) for a in (k, v, q))
    g = c["QH"] // c["KVH"]
    out = np.zeros((c["QH"], c["D"]))
    for h in range(c["QH"]):
        s = kf[:, h // g, :] @ qf[h] / np.sqrt(c["D"])
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ vf[:, h // g, :]
    return {"config": c, "scale": 1.0 / float(np.sqrt(c["D"])), "inputs_sha256": inputs_digest(table, k, v, q),
            "table": table.tolist(), "out_f32": [[float(np.float32(x)) for x in row] for row in out]}


# ---- E4M3FN -------------------------------------------------------------------------
def e4m3fn_value(code):
    s, e, m = code >> 7, (code >> 3) & 15, code & 7
    if e == 15 and m == 7:
        return None
    mag = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
    return -mag if s else mag


def e4m3fn():
    values = [e4m3fn_value(c) for c in range(256)]
    pos = [(values[c], c) for c in range(0x7F)]                 # 0 .. 448, increasing with the code
    cases = [[v, c] for v, c in pos] + [[-v, c | 0x80] for v, c in pos]
    for (a, ca), (b, cb) in zip(pos[:-1], pos[1:]):
        mid = (a + b) / 2                                        # exact in fp32: at most 5 significant bits
        even = ca if ca % 2 == 0 else cb
        cases.append([mid, even])
        cases.append([-mid, even | 0x80])
        lo = float(np.nextafter(np.float32(mid), np.float32(-np.inf)))
        hi = float(np.nextafter(np.float32(mid), np.float32(np.inf)))
        cases.append([lo, ca])
        cases.append([hi, cb])
    # by this build's specification: values beyond +-448, infinities included, saturate
    for v in (448.5, 464.0, 480.0, 1.0e30):
        cases.append([v, 0x7E])
        cases.append([-v, 0xFE])
    return {"values": values, "encode": cases, "saturating": {"inf": 0x7E, "-inf": 0xFE}}


# ---- int8 rows ------------------------------------------------------------------------
def int8_row(x16):
    """x16: fp16 values (the source row).  Every step in IEEE arithmetic of the stated width."""
    x = x16.astype(np.float32)
    amax = np.float32(np.max(np.abs(x))) if len(x) else np.float32(0)
    s32 = np.float32(amax) / np.float32(127.0)
    sh = np.float16(s32)
    if np.isinf(sh):
        sh = np.float16(65504.0)
    sf = np.float32(sh)
    rcp = np.float32(1.0) / sf if sf > 0 else np.float32(0.0)
    t = (x * rcp).astype(np.float32)
    codes = np.clip(np.rint(t), -127, 127).astype(np.int8)       # numpy's rint rounds half to even
    return int(np.array(sh).view(np.uint16)), codes.tolist()


def int8_rows():
    rows = []
    ties = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5, -126.5, 63.5, 64.5, 0.25, 0.75, -0.0, 0.0], np.float16)
    rows.append(ties)                                            # scale exactly 1: the .5 ties show
    rows.append(np.zeros(16, np.float16))                        # all zero: scale 0, codes 0
    rows.append(np.array([65504.0, -65504.0, 1.0, 300.0] * 4, np.float16))
    rows.append(np.array([6.1e-5, -6.1e-5, 3e-5, 5.96e-8] * 4, np.float16))      # around fp16 subnormals
    rows.append((normals(128, 77) * 0.5).astype(np.float16))
    big = (normals(128, 78)).astype(np.float16)
    big[[3, 90]] = np.float16(20.0) * big[[3, 90]]
    rows.append(big)
    rows.append(np.array([254.0, 1.0, 3.0, 5.0, 253.0, -251.0, 127.0, -129.0], np.float16))   # scale 2: x/2 ties
    out = []
    for r in rows:
        scale_bits, codes = int8_row(r)
        out.append({"x_f16_bits": r.view(np.uint16).tolist(), "scale_f16_bits": scale_bits, "codes": codes})
    return {"rows": out}


# ---- BlockPool free stack -------------------------------------------------------------
def block_pool_trace():
    nb = 6
    free = list(range(nb - 1, -1, -1))                           # back of the list = next id: 0, 1, 2, ...
    ops, script = [], [("alloc",)] * 4 + [("free", 1), ("free", 3), ("alloc",), ("alloc",), ("alloc",), ("alloc",),
                                          ("alloc",), ("free", 0), ("free", 5), ("free", 2), ("alloc",), ("alloc",),
                                          ("alloc",), ("alloc",)]
    for op in script:
        if op[0] == "alloc":
            got = free.pop() if free else -1
            ops.append({"op": "alloc", "returns": got, "free_count": len(free)})
        else:
            free.append(op[1])
            ops.append({"op": "free", "id": op[1], "free_count": len(free)})
    return {"max_blocks": nb, "ops": ops}


def main():
    for name, obj in (("e4m3fn_table.json", e4m3fn()), ("int8_rows.json", int8_rows()),
                      ("block_pool_trace.json", block_pool_trace()), ("config1_decode.json", config1())):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(obj, f, separators=(",", ":"))
            f.write("\n")
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
