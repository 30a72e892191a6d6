"""Writes tests/golden/ring_cases.npz: small input / expected-output vectors for the ring collectives and the
reduce-copy primitive, produced by the CPU oracle (the reference holds no vectors for this path and cannot be
built or run here).  They freeze the oracle's behaviour: the CPU suite checks that the oracle still reproduces
them, the GPU suite that the HIP path does.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
sys.path.insert(0, os.path.join(HERE, ".."))

import datagen  # noqa: E402
import dfccl_oracle as orc  # noqa: E402

# kind, dtype, op, n, count, root, (nChannels, chunkElems, alignElems)
# The float all-reduce cases use the geometry the library plans for these sizes (one channel, 8 KiB chunks,
# 1 KiB rounding), so that the GPU suite can compare them bit for bit.
CASES = [
    ("all_reduce", orc.F32, orc.SUM, 2, 1000, 0, (1, 2048, 256)),
    ("all_reduce", orc.F32, orc.SUM, 4, 2048, 0, (1, 2048, 256)),
    ("all_reduce", orc.BF16, orc.SUM, 8, 4100, 0, (1, 4096, 512)),
    ("all_reduce", orc.F16, orc.SUM, 4, 2048, 0, (1, 4096, 512)),
    ("all_reduce", orc.F16, orc.PROD, 3, 777, 0, (1, 4096, 512)),
    ("all_reduce", orc.I32, orc.SUM, 5, 1234, 0, (2, 256, 256)),
    ("all_reduce", orc.I8, orc.MIN, 4, 5000, 0, (1, 1024, 1024)),
    ("all_reduce", orc.F32, orc.MAX, 8, 900, 0, (1, 256, 256)),
    ("all_reduce", orc.BF16, orc.PROD, 2, 513, 0, (1, 4096, 512)),
    ("reduce_scatter", orc.F32, orc.SUM, 4, 700, 0, (1, 256, 256)),
    ("reduce_scatter", orc.BF16, orc.SUM, 3, 1025, 0, (2, 512, 512)),
    ("reduce_scatter", orc.I8, orc.MAX, 8, 300, 0, (1, 1024, 1024)),
    ("all_gather", orc.F16, orc.SUM, 4, 333, 0, (1, 1024, 1024)),
    ("all_gather", orc.I32, orc.SUM, 3, 1000, 0, (2, 1024, 1024)),
    ("reduce", orc.F32, orc.SUM, 4, 999, 2, (1, 256, 256)),
    ("reduce", orc.F16, orc.MIN, 5, 1500, 0, (1, 512, 512)),
    ("broadcast", orc.BF16, orc.SUM, 4, 1111, 3, (1, 1024, 1024)),
    ("reduce_copy", orc.F32, orc.SUM, 2, 4097, 0, None),
    ("reduce_copy", orc.BF16, orc.SUM, 3, 1000, 0, None),
    ("reduce_copy", orc.I8, orc.PROD, 4, 2000, 0, None),
    ("reduce_copy", orc.F16, orc.MAX, 8, 515, 0, None),
    # the remaining element types and the scaled sums (appended: the cases above keep their numbers and inputs)
    ("all_reduce", orc.U8, orc.MAX, 4, 3000, 0, (1, 8192, 1024)),
    ("all_reduce", orc.U32, orc.SUM, 3, 1500, 0, (1, 2048, 256)),
    ("all_reduce", orc.I64, orc.MIN, 4, 900, 0, (1, 1024, 128)),
    ("all_reduce", orc.U64, orc.PROD, 2, 600, 0, (1, 1024, 128)),
    ("all_reduce", orc.F64, orc.SUM, 4, 900, 0, (1, 1024, 128)),
    ("all_reduce", orc.I32, orc.AVG, 5, 1234, 0, (1, 2048, 256)),
    ("all_reduce", orc.U8, orc.AVG, 3, 2000, 0, (1, 8192, 1024)),
    ("all_reduce", orc.BF16, orc.AVG, 4, 2048, 0, (1, 4096, 512)),
    ("all_reduce", orc.F32, orc.AVG, 8, 4000, 0, (1, 2048, 256)),
    ("reduce_scatter", orc.I64, orc.AVG, 4, 300, 0, (1, 1024, 128)),
    ("reduce", orc.F64, orc.AVG, 3, 700, 1, (1, 1024, 128)),
    ("reduce_copy", orc.U32, orc.AVG, 5, 1000, 0, None),
    ("reduce_copy", orc.F16, orc.AVG, 3, 1000, 0, None),
]

# PreMulSum with every rank's own scalar (rank r's input enters the sum times VALUES[r]):
# kind, dtype, values per rank, n, count, root, geometry.  Arrays p<idx>_in<r> / p<idx>_out<r>.
PREMUL_CASES = [
    ("all_reduce", orc.F32, [0.3, -1.7, 2.5, 0.01], 4, 2048, 0, (1, 2048, 256)),
    ("all_reduce", orc.BF16, [-1.5, 0.5, 2.0, -0.25, 1.0, 3.0, -2.0, 0.75], 8, 4100, 0, (1, 4096, 512)),
    ("all_reduce", orc.I32, [1000003, -3, 7], 3, 1500, 0, (1, 2048, 256)),
    ("all_reduce", orc.F64, [1e-3, -2.5], 2, 600, 0, (1, 1024, 128)),
    ("reduce_scatter", orc.F16, [0.5, -1.25, 2.0, 0.1], 4, 700, 0, (1, 512, 512)),
    ("reduce", orc.U8, [3, 2, 5], 3, 2000, 1, (1, 8192, 1024)),
]


def premul_bits(dtype, values):
    return [orc.scalar_bits(dtype, v) for v in values]


def run_premul_case(kind, dtype, values, n, count, root, geom, sends):
    g = orc.Geom(n, *geom)
    bits = premul_bits(dtype, values)
    if kind == "all_reduce":
        return orc.all_reduce(dtype, orc.PREMULSUM, g, sends, scalar=bits)
    if kind == "reduce_scatter":
        return orc.reduce_scatter(dtype, orc.PREMULSUM, g, sends, scalar=bits)
    return orc.reduce(dtype, orc.PREMULSUM, g, root, sends, scalar=bits)


def run_case(kind, dtype, op, n, count, root, geom, sends):
    if kind == "reduce_copy":
        return [orc.reduce_copy(dtype, op, sends)]
    g = orc.Geom(n, *geom)
    if kind == "all_reduce":
        return orc.all_reduce(dtype, op, g, sends)
    if kind == "reduce_scatter":
        return orc.reduce_scatter(dtype, op, g, sends)
    if kind == "all_gather":
        return orc.all_gather(dtype, g, sends)
    if kind == "reduce":
        return orc.reduce(dtype, op, g, root, sends)
    return orc.broadcast(dtype, g, root, sends)


def make_inputs(kind, dtype, op, n, count, idx):
    length = count * n if kind == "reduce_scatter" else count
    return [datagen.make(dtype, 9000 + 16 * idx + r, length, small_ints=(op == orc.PROD)) for r in range(n)]


def main():
    out = {}
    for idx, (kind, dtype, op, n, count, root, geom) in enumerate(CASES):
        sends = make_inputs(kind, dtype, op, n, count, idx)
        recvs = run_case(kind, dtype, op, n, count, root, geom, sends)
        for r, a in enumerate(sends):
            out[f"c{idx}_in{r}"] = a
        for r, a in enumerate(recvs):
            out[f"c{idx}_out{r}"] = a
    for idx, (kind, dtype, values, n, count, root, geom) in enumerate(PREMUL_CASES):
        length = count * n if kind == "reduce_scatter" else count
        sends = [datagen.make(dtype, 12000 + 16 * idx + r, length) for r in range(n)]
        recvs = run_premul_case(kind, dtype, values, n, count, root, geom, sends)
        for r, a in enumerate(sends):
            out[f"p{idx}_in{r}"] = a
        for r, a in enumerate(recvs):
            out[f"p{idx}_out{r}"] = a
    np.savez_compressed(os.path.join(HERE, "ring_cases.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
