"""CPU oracle, the .nc data path -- TEST INFRASTRUCTURE ONLY (only tests/ may import this).

numpy restatement of /root/reference/CURRENNT_codes/currennt_lib/src/data_sets/DataSet.cpp:
  :1376-1500  per file: first max(1, int(numSeqs*fraction)) sequences; a sequence longer than 1.5*truncSeqLength
              is cut into segments of truncSeqLength, the remainder staying with the last one
  :1831-1832  segments are consecutive row ranges of inputs / targetPatterns / targetClasses
  :1897-1900  training mode: segments sorted by ascending length
  :642-1022   _makeFractionTask: slot t*S+i of a fraction holds step t of its i-th segment; padding slots hold
              zero inputs / targets, class -1 and patType NONE; patTypes FIRST(1) / NORMAL(2) / LAST(3)
The file itself is read with scipy.io.netcdf_file, the library the reference's own tooling writes these files
with (pyTools/dataTools/ncDataHandle.py:174-186).
"""
import numpy as np
from scipy.io import netcdf_file


def segments(path, fraction=1.0, truncate_seq=0, training_mode=True):
    f = netcdf_file(path, "r", mmap=False)
    n_seq = f.dimensions["numSeqs"]
    take = max(int(np.float32(n_seq) * np.float32(fraction)), 1)
    lengths = [int(v) for v in f.variables["seqLengths"][:take]]
    tags = [b"".join(row).split(b"\0")[0].decode() for row in f.variables["seqTags"][:take]]
    f.close()
    out, begin = [], 0
    for length, tag in zip(lengths, tags):
        k, remaining = 0, length
        while remaining > 0:
            seg = min(truncate_seq, remaining) if (truncate_seq > 0 and remaining > 1.5 * truncate_seq) else remaining
            out.append({"length": seg, "begin": begin, "tag": tag, "original_seq_idx": k})
            begin += seg
            remaining -= seg
            k += 1
    if training_mode:
        out.sort(key=lambda s: s["length"])  # Python's sort is stable
    return out


def make_fraction(path, segs, first_seq, S):
    f = netcdf_file(path, "r", mmap=False)
    P = f.dimensions["inputPattSize"]
    is_cls = "numLabels" in f.dimensions
    Q = (1 if f.dimensions["numLabels"] == 2 else f.dimensions["numLabels"]) if is_cls else f.dimensions["targetPattSize"]
    part = segs[first_seq:first_seq + S]
    T = max(s["length"] for s in part)
    pat = np.zeros(T * S, np.int8)
    x = np.zeros((T * S, P), np.float32)
    tgt = None if is_cls else np.zeros((T * S, Q), np.float32)
    cls = np.full(T * S, -1, np.int32) if is_cls else None
    for i, s in enumerate(part):
        for t in range(s["length"]):
            slot = t * S + i
            x[slot] = f.variables["inputs"][s["begin"] + t]
            if is_cls:
                cls[slot] = f.variables["targetClasses"][s["begin"] + t]
            else:
                tgt[slot] = f.variables["targetPatterns"][s["begin"] + t]
            pat[slot] = 1 if t == 0 else (3 if t == s["length"] - 1 else 2)
    f.close()
    return {"num_seqs": len(part), "max_len": T, "min_len": min(s["length"] for s in part),
            "total_length": sum(s["length"] for s in part), "patTypes": pat, "inputs": x.reshape(-1),
            "targets": None if tgt is None else tgt.reshape(-1), "target_classes": cls}
