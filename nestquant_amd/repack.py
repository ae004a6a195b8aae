"""Published shards -> the files a serving rank reads: one record file per tensor-parallel rank + its resident planes.

    python -m nestquant_amd.repack ROOT OUT [tp=4] [layers=3-77] [rec_bytes]

Host-side mirror of the reference's streaming/repack.py (same arguments, file names and index keys, so either side's
output serves the other):
    OUT/rank{r}.bin          record of (layer L, expert E) at ((L - L0) * NE + E) * rec_bytes; rec_bytes is the same for every
                             layer (4 KiB aligned, the slot size), so layers can be written in any order
    OUT/rank{r}.json         {format 'nq-p4rec-v1', tp, rank, L0, NE, rec_bytes, seg {segment: [offset, bytes]},
                             layers {L: {experts [ids], rg {id: rank}, rd {id: rank}}}}
    OUT/res/rank{r}/L{L}.pt  the layer's resident planes (resident.py)
Layers already written are skipped, layers whose shards are not all there yet are reported and left for a later run;
several runs may work on different layers at once (the index is merged under a file lock).

`record_offset` and `read_record` are the reader's half: where a record lies, and one positioned read of it into a
caller's buffer (for instance the pinned staging buffer a promotion copies from).
"""
import fcntl
import json
import os
import sys
import time

import torch

from . import nqload, p4rec, resident

NE = 256
L0 = 3
FORMAT = "nq-p4rec-v1"


def parse_layers(s):
    """'7' -> [7]; '3-77' -> [3, ..., 77]"""
    a, b = (s.split("-") + [s])[:2]
    return list(range(int(a), int(b) + 1))


def _have_shards(d):
    return os.path.exists(f"{d}/manifest.json") and all(
        os.path.exists(f"{d}/tp{i}.pt") or os.path.exists(f"{d}/tp{i}.safetensors") for i in range(nqload.NSH))


def _read_index(path, tp, rank, ne, l0):
    if os.path.exists(path):
        with open(path) as f:
            return json.load(f)
    return dict(format=FORMAT, tp=tp, rank=rank, L0=l0, NE=ne, layers={})


def record_offset(idx, L, E):
    """byte offset of the record of (layer L, expert E) in the rank's record file, from its index"""
    return ((L - idx["L0"]) * idx["NE"] + E) * idx["rec_bytes"]


def read_record(fd, idx, L, E, buf):
    """one positioned read of the record of (L, E) from the open record file `fd` into `buf` (a flat CPU uint8 tensor of at
    least rec_bytes elements, pinned or not); returns the filled part"""
    n = idx["rec_bytes"]
    if buf.dtype != torch.uint8 or buf.dim() != 1 or buf.numel() < n or buf.device.type != "cpu":
        raise ValueError("read_record needs a flat CPU uint8 tensor of at least rec_bytes elements")
    if str(L) not in idx["layers"] or E not in idx["layers"][str(L)]["experts"]:
        raise KeyError(f"no record of layer {L}, expert {E} in this file")
    got = os.preadv(fd, [memoryview(buf.numpy())[:n]], record_offset(idx, L, E))
    if got != n:
        raise IOError(f"record of layer {L}, expert {E}: {got} of {n} bytes")
    return buf[:n]


def repack(root, out, tp=4, layers=None, rec_bytes=None, dev="cuda", ne=NE, l0=L0, log=print):
    """write the records and resident files of `layers` (default 3..77) for every rank of a tensor-parallel run of degree tp;
    returns the list of (layer, rank) written by this call"""
    layers = list(range(3, 78)) if layers is None else list(layers)
    os.makedirs(out, exist_ok=True)
    done = []
    for L in layers:
        d = nqload.layer_dir(root, L)
        if not _have_shards(d):
            log(f"L{L}: not fitted / downloaded yet")
            continue
        for r in range(tp):
            ip = f"{out}/rank{r}.json"
            idx = _read_index(ip, tp, r, ne, l0)
            rp = f"{out}/res/rank{r}/L{L}.pt"
            os.makedirs(os.path.dirname(rp), exist_ok=True)
            if str(L) in idx["layers"] and os.path.exists(rp):
                continue
            t0 = time.time()
            RL = nqload.RankLayer(root, L, r, tp, dev=dev)
            if not os.path.exists(rp):
                resident.save(RL, rp)
                log(f"L{L} rank{r}: resident planes {os.path.getsize(rp) / 2**20:.0f} MiB")
            if str(L) in idx["layers"]:
                continue
            lay = p4rec.layout(next(iter(RL.ex.values())), RL.H, RL.I)
            seg = {k: list(v) for k, v in lay["seg"].items()}
            if "rec_bytes" not in idx:
                idx["rec_bytes"] = int(rec_bytes) if rec_bytes else lay["rec_bytes"]
                idx["seg"] = seg
            if seg != idx["seg"] or lay["rec_bytes"] > idx["rec_bytes"]:
                raise ValueError(f"layer {L}: record layout {seg}, {lay['rec_bytes']} B does not fit the file's "
                                 f"{idx['seg']}, {idx['rec_bytes']} B")
            if any(E >= idx["NE"] for E in RL.experts) or L < idx["L0"]:
                raise ValueError(f"layer {L}: expert ids {RL.experts} / layer index outside the file's NE = {idx['NE']}, L0 = {idx['L0']}")
            lay["rec_bytes"] = rb = idx["rec_bytes"]
            fd = os.open(f"{out}/rank{r}.bin", os.O_WRONLY | os.O_CREAT, 0o644)
            try:
                for E, ex in RL.ex.items():
                    os.pwrite(fd, p4rec.pack(ex, lay), record_offset(idx, L, E))
                os.fsync(fd)
            finally:
                os.close(fd)
            ent = dict(experts=RL.experts, rg={str(E): RL.ex[E].rg for E in RL.experts}, rd={str(E): RL.ex[E].rd for E in RL.experts})
            with open(f"{out}/rank{r}.lock", "w") as lk:     # merge with what other runs added meanwhile
                fcntl.flock(lk, fcntl.LOCK_EX)
                cur = _read_index(ip, tp, r, ne, l0)
                cur.setdefault("rec_bytes", idx["rec_bytes"])
                cur.setdefault("seg", idx["seg"])
                cur["layers"][str(L)] = ent
                tmp = f"{ip}.{os.getpid()}.tmp"
                with open(tmp, "w") as f:
                    json.dump(cur, f)
                os.replace(tmp, ip)
            log(f"L{L} rank{r}: {len(RL.experts)} records x {rb} B in {time.time() - t0:.1f}s")
            done.append((L, r))
            del RL
    return done


def main(argv=None):
    a = sys.argv[1:] if argv is None else argv
    if len(a) < 2:
        print(__doc__)
        return 2
    repack(a[0], a[1], tp=int(a[2]) if len(a) > 2 else 4, layers=parse_layers(a[3]) if len(a) > 3 else None,
           rec_bytes=int(a[4]) if len(a) > 4 else None)
    return 0


if __name__ == "__main__":
    sys.exit(main())
