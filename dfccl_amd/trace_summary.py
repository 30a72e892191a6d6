"""Summary of a device timeline written by the library (DFCCL_TRACE=1, DFCCL_TRACE_FILE=<file>).

The file holds, for every workgroup (rank slot x channel, 16 x 64 of them), 4096 records of two 64-bit words:
event | arg << 32 and a 100 MHz tick; the last record slot of a workgroup holds how many records it wrote.

    python -m dfccl_amd.trace_summary <file> <channels per rank> [<rank slots>]
    python -m dfccl_amd.trace_summary --steps <file> <workgroup>[,<workgroup>...]

prints, for the last instance every workgroup moved data for, when (in microseconds after the first submission
of that instance was fetched) the submissions were fetched and ingested, the data movement began and ended, the
completions were posted and the visits ended: minimum, median and maximum over the workgroups.  With --steps:
for each of the given workgroups, every record from a fetch to the end of the visit that follows it, as
microseconds after the fetch (median / minimum / 90th percentile over all instances with the same sequence of
events): the step-by-step cost of one small collective."""
import sys

import numpy as np

EVENTS = {1: "sqeFetched", 2: "ingested", 3: "visitBegin", 4: "waitBegin", 5: "waitEnd", 6: "moveBegin", 7: "moveEnd",
          8: "posted", 9: "cqePosted", 10: "visitEnd", 11: "scanDone", 12: "launch", 13: "exit", 14: "roundDecided",
          15: "runEntry", 16: "laidOut", 17: "folded", 18: "runReturned"}
RECORDS, MAX_CHANNELS = 4096, 64


def last_instance(records):
    """Times of the events around the last moveBegin of one workgroup."""
    n = int(records[RECORDS - 1, 1])
    rec = records[:min(n, RECORDS - 1)]
    ev = (rec[:, 0] & 0xffffffff).astype(int)
    t = rec[:, 1].astype(np.int64)
    begins = np.nonzero(ev == 6)[0]
    if len(begins) == 0:
        return None
    i = begins[-1]
    out = {"moveBegin": t[i]}
    for j in range(i, -1, -1):
        if ev[j] == 2 and "ingested" not in out:
            out["ingested"] = t[j]
        if ev[j] == 1:
            out["sqeFetched"] = t[j]
            break
    for j in range(i, len(ev)):
        name = EVENTS.get(ev[j])
        if name in ("moveEnd", "cqePosted") and name not in out:
            out[name] = t[j]
        if ev[j] == 10:
            out["visitEnd"] = t[j]
            break
    return out


def steps(path, wgs):
    a = np.fromfile(path, dtype=np.uint64).reshape(-1, RECORDS, 2)
    for wg in wgs:
        n = int(a[wg, RECORDS - 1, 1])
        rec = a[wg, :min(n, RECORDS - 1)]
        ev = (rec[:, 0] & 0xffffffff).astype(int)
        t = rec[:, 1].astype(np.int64)
        seqs = {}
        for s in np.nonzero(ev == 1)[0][5:]:  # (the first few instances are warm-up)
            names, times = [], []
            for j in range(s, len(ev)):
                names.append(EVENTS.get(ev[j], str(ev[j])))
                times.append((t[j] - t[s]) / 100.0)
                if ev[j] == 10:
                    break
            seqs.setdefault(tuple(names), []).append(times)
        print(f"workgroup {wg}: {n} records")
        for key, v in sorted(seqs.items(), key=lambda kv: -len(kv[1]))[:2]:
            arr = np.array(v)
            print(f"  {len(v)} instances with this sequence (median / min / p90, us after the fetch):")
            for i, name in enumerate(key):
                print(f"    {name:11s} {np.median(arr[:, i]):7.2f} {arr[:, i].min():7.2f} {np.percentile(arr[:, i], 90):7.2f}")
    return 0


def main(argv):
    if len(argv) > 3 and argv[1] == "--steps":
        return steps(argv[2], [int(x) for x in argv[3].split(",")])
    path, channels = argv[1], int(argv[2])
    slots = int(argv[3]) if len(argv) > 3 else 16
    a = np.fromfile(path, dtype=np.uint64).reshape(-1, RECORDS, 2)
    rows = []
    for slot in range(slots):
        for ch in range(channels):
            # records are stored by slot * launched channels + channel; the launch rounds channels up to 8
            wg = slot * ((channels + 7) // 8 * 8 if channels > 1 else 1) + ch
            if wg < a.shape[0]:
                r = last_instance(a[wg])
                if r:
                    rows.append(r)
    if not rows:
        print("no data movement recorded")
        return 1
    t0 = min(r["sqeFetched"] for r in rows if "sqeFetched" in r)
    print(f"{len(rows)} workgroups; microseconds after the first submission was fetched (min / median / max)")
    for key in ("sqeFetched", "ingested", "moveBegin", "moveEnd", "cqePosted", "visitEnd"):
        v = np.array([(r[key] - t0) / 100.0 for r in rows if key in r])
        if len(v):
            print(f"  {key:11s} n={len(v):4d}  {v.min():9.2f} {np.median(v):9.2f} {v.max():9.2f}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
