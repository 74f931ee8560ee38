"""LDS bank conflicts of the address patterns the tile kernels use, and which lanes an LDS instruction serves together.

    rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS --kernel-trace --output-format csv \\
        -d /tmp/lds_probe -o p -- python3 -m tritonix_amd.lds_probe
    python3 -m tritonix_amd.lds_probe --counters /tmp/lds_probe/<host>/p_counter_collection.csv

The first command launches ``tnx_probe_lds`` once per pattern below (one wave, 16000 instructions each); the second
reads the counters of those dispatches, in order, and prints conflict and active cycles per instruction.  The
"pair" patterns find the lanes that share a cycle: every lane reads one common address except a reference lane and
one other lane, which read different addresses on the same banks -- they conflict only if served together.
"""
import ctypes
import sys

from . import _C


def swz_a(row, wide=True, old=False):
    if old:
        return ((row & 7) ^ ((row >> 3) & 1)) if wide else (((row >> 1) & 3) ^ ((row >> 3) & 1))
    return ((row & 7) ^ ((row >> 2) & 1)) if wide else (((row >> 3) & 1) << 1)


def a_fragment(pitch, kstep=0, row0=0, old=False):
    """ds_read_b128 of an A fragment: lane = 16 * kg + row, 16-byte chunk (kstep * 4 + kg) ^ swizzle(row)."""
    chunks = pitch // 16
    return [(row0 + l % 16) * pitch + ((((kstep * 4 + l // 16) % chunks) ^ swz_a(row0 + l % 16, pitch >= 128, old)) << 4)
            for l in range(64)]


def b_fragment(es):
    """Transposing read of a B fragment from a slab with BN = 256 (rows of 512 resp. 256 bytes), column block 0."""
    out = []
    for l in range(64):
        blk, li = l >> 4, l & 15
        sub, col = (li >> 2, 8 * (li & 3)) if es == 2 else (li >> 1, 8 * (li & 1))
        row = (16 // es) * blk + sub
        if es == 2:
            k = row & 3
            sw = ((2 * k + (k >> 1)) << 1) ^ ((((row >> 3) ^ (row >> 4)) & 1) << 1)
        else:
            k = row & 7
            sw = (2 * k + (k >> 2)) ^ (((row >> 4) ^ (row >> 5)) & 1)
        out.append(row * 256 * es + (((col >> 4) ^ sw) << 4) + (col & 15))
    return out


def pair(ref, other):
    return [256 + 64 if l == ref else (512 + 64 if l == other else 16) for l in range(64)]


def patterns():
    p = [("A fragment, 128-byte rows, swizzle in use", _C.LDS_READ_B128, a_fragment(128)),
         ("A fragment, 128-byte rows, k step 1, rows 16-31", _C.LDS_READ_B128, a_fragment(128, 1, 16)),
         ("A fragment, 128-byte rows, previous swizzle", _C.LDS_READ_B128, a_fragment(128, old=True)),
         ("A fragment, 64-byte rows, swizzle in use", _C.LDS_READ_B128, a_fragment(64)),
         ("A fragment, 64-byte rows, previous swizzle", _C.LDS_READ_B128, a_fragment(64, old=True)),
         ("A fragment, no swizzle", _C.LDS_READ_B128, [(l % 16) * 128 + (l // 16) * 16 for l in range(64)]),
         ("linear, lane * 16", _C.LDS_READ_B128, [l * 16 for l in range(64)]),
         ("B fragment bf16 (ds_read_b64_tr_b16), swizzle in use", _C.LDS_READ_TR16_B64, b_fragment(2)),
         ("B fragment int8 (ds_read_b64_tr_b8), swizzle in use", _C.LDS_READ_TR8_B64, b_fragment(1)),
         ("epilogue strip write, pitch 528", _C.LDS_WRITE_B128, [(l % 16) * 528 + (l // 16) * 16 for l in range(64)])]
    for op, name in ((_C.LDS_READ_B128, "ds_read_b128"), (_C.LDS_WRITE_B128, "ds_write_b128")):
        for ref in (0, 4):
            p += [(f"pair {name} lane {ref} with lane {o}", op, pair(ref, o)) for o in range(32) if o != ref]
    return p


def run():
    import torch
    scratch = torch.zeros(128, dtype=torch.int32, device="cuda:0")
    lib = _C.load()
    for i, (name, op, offs) in enumerate(patterns()):
        table = (ctypes.c_uint32 * 64)(*offs)
        st = lib.tnx_probe_lds(op, table, 2000, scratch.data_ptr(), 512, torch.cuda.current_stream().cuda_stream)
        if st != _C.OK:
            raise RuntimeError(f"tnx_probe_lds: {_C.strerror(st)} for pattern {name}")
        torch.cuda.synchronize()
        print(f"dispatch {i}: {name}")


def report(path):
    import csv
    rows = {}
    for r in csv.DictReader(open(path)):
        if "lds_pattern_kernel" in r["Kernel_Name"]:
            rows.setdefault(int(r["Dispatch_Id"]), {})[r["Counter_Name"]] = float(r["Counter_Value"])
    disp = [rows[k] for k in sorted(rows)]
    pats = patterns()
    if len(disp) != len(pats):
        raise SystemExit(f"{len(disp)} probe dispatches in {path}, {len(pats)} patterns here")
    groups = {}
    for (name, _, _), c in zip(pats, disp):
        n = max(c["SQ_INSTS_LDS"], 1.0)
        conflict, active = c["SQ_LDS_BANK_CONFLICT"] / n, c["SQ_LDS_IDX_ACTIVE"] / n
        if name.startswith("pair"):
            w = name.split()
            if conflict > 0.4:
                groups.setdefault((w[1], int(w[3])), []).append(int(w[6]))
        else:
            print(f"{name:58s} conflict cycles / instruction {conflict:5.2f}   active {active:5.2f}")
    for (op, ref), lanes in sorted(groups.items()):
        print(f"{op}: lane {ref} shares its cycle with lanes {lanes} (of lanes 0-31)")


if __name__ == "__main__":
    if len(sys.argv) == 3 and sys.argv[1] == "--counters":
        report(sys.argv[2])
    elif len(sys.argv) == 1:
        run()
    else:
        raise SystemExit(__doc__)
