"""Ring-order results of the collectives restated in torch tensor operations (test infrastructure).

An independent check for inputs too large for the CPU oracle: the chunk -> owner geometry is written out in
torch integer arithmetic, and a chunk owned by rank c is folded in[c+1], in[c+2], ..., in[c] with torch's own
add / mul / max / min in the storage type (one rounding per step: torch computes a bf16 or fp16 operation in
fp32 and rounds the result to nearest even, which equals the correctly rounded operation of the storage type).
The ring accumulates a chunk in that order on its way to the owner
(src/collectives_ofccl/device/ofccl_all_reduce.h:58-63,76-171 of the reference).  tests/test_torch_ring_cpu.py
pins this restatement against the CPU oracle at sizes the oracle covers; it runs on whatever device the inputs
are on.
"""
import torch

OPS = {
    "sum": torch.add,
    "prod": torch.mul,
    "max": torch.maximum,
    "min": torch.minimum,
}


def _div_up(a, b):
    return (a + b - 1) // b


def all_reduce_owner_map(count, n, channels, chunk, align, device):
    """int64 tensor: rank that owns element i (the rank at which the ring's reduce-scatter half ends for it).

    Loops of channels * n chunks; every loop uses the nominal chunk except the last, which splits what is left
    evenly (rounded up to `align`); inside a loop chunk k belongs to channel k // n and rank k % n."""
    loop = channels * n * chunk
    nloops = _div_up(count, loop)
    last_start = (nloops - 1) * loop
    last_real = _div_up(min(chunk, _div_up(count - last_start, channels * n)), align) * align
    i = torch.arange(count, device=device, dtype=torch.int64)
    l = torch.div(i, loop, rounding_mode="floor")
    j = i - l * loop
    real = torch.where(l == nloops - 1, torch.full_like(i, last_real), torch.full_like(i, chunk))
    return torch.div(j, real, rounding_mode="floor") % n


def fold_in_ring_order(sends, owner, op="sum"):
    """out[i] = sends[c+1][i] (op) sends[c+2][i] (op) ... (op) sends[c][i] with c = owner[i], left to right."""
    n = len(sends)
    f = OPS[op]
    out = torch.empty_like(sends[0])
    for c in range(n):
        idx = (owner == c).nonzero(as_tuple=True)[0]
        if idx.numel() == 0:
            continue
        acc = sends[(c + 1) % n][idx]
        for j in range(2, n + 1):
            acc = f(acc, sends[(c + j) % n][idx])
        out[idx] = acc
    return out


def all_reduce_expected(sends, geom, op="sum"):
    """geom: object with nRanks, nChannels, chunkElems, alignElems (what dfcclGetCollGeometry reports)."""
    count = sends[0].numel()
    owner = all_reduce_owner_map(count, geom.nRanks, geom.nChannels, geom.chunkElems, geom.alignElems,
                                 sends[0].device)
    return fold_in_ring_order(sends, owner, op)


def same_bits(a, b):
    """Bit-for-bit equality of two tensors of the same dtype (floats compared as integers)."""
    if a.dtype in (torch.bfloat16, torch.float16):
        return torch.equal(a.view(torch.int16), b.view(torch.int16))
    if a.dtype == torch.float32:
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    if a.dtype == torch.float64:
        return torch.equal(a.view(torch.int64), b.view(torch.int64))
    return torch.equal(a, b)
