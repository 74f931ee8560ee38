"""Build libtritonix_hip.so (gfx950) from tritonix_amd/csrc with hipcc.

    python -m tritonix_amd.build [--jobs N] [--quick] [--only TILES --out PATH -D MACRO]

The tile kernels are C++ templates; this script writes one small instance
file per (dtype, block_m) group into build/gen/, compiles the groups in
parallel and links everything into tritonix_amd/libtritonix_hip.so.  The
shared object is what travels to a GPU machine; nothing is compiled there.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import glob
import json
import os
import re
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(ROOT, "build")
LIB = os.path.join(HERE, "libtritonix_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 VALU ops are switched off on purpose for every device translation unit
DEVICE_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                # the K loop is written as fully unrolled slots; with the conv2d loader in them the default limit on
                # the size of a pragma-unrolled loop would leave one rolled (and the accumulators in scratch memory)
                "-mllvm", "-pragma-unroll-threshold=100000",
                "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]

LDS_LIMIT = 160 * 1024
TAGS = {"bf16": ("TagBF16", 2), "f16": ("TagF16", 2), "i8": ("TagI8", 1)}


def tile_valid(es, bm, bn, bk, nw, stages):
    """Mirror of TileCfg::VALID in csrc/gemm_tile.h."""
    wgm = 2 if nw == 4 else (4 if bm > bn else 2)
    wgn = nw // wgm
    if bm % wgm or bn % wgn:
        return False
    wtm, wtn = bm // wgm, bn // wgn
    if wtm % 16 or wtn % 16:
        return False
    mi = 16                      # TileCfg::MI: the 16x16 MFMA shapes everywhere
    tm, tn = wtm // mi, wtn // mi
    kb = 32 if mi == 32 else 64
    if (bk * es) % kb or bk * es < kb:
        return False
    cpr_a, cpr_b = bk * es // 16, bn * es // 16
    if cpr_a < 4 or cpr_b < 8 or cpr_b % (4 if es == 1 else 8):
        return False
    a_bytes, b_bytes = bm * bk * es, bk * bn * es
    if a_bytes % 1024 or b_bytes % 1024:
        return False
    a_loads, b_loads = a_bytes // 1024, b_bytes // 1024
    if a_loads % nw or b_loads % nw:
        return False
    lpw = a_loads // nw + b_loads // nw
    if stages < 2 or (stages - 2) * lpw > 63:
        return False
    if stages * (a_bytes + b_bytes) > LDS_LIMIT:
        return False
    if tm * tn * (16 if mi == 32 else 4) > 256:
        return False
    return True


def parse_only(spec):
    """'bf16:256:256:64:4:2,i8:256:256:128:4:2' -> instance tuples (development builds of a few tiles)."""
    out = []
    for item in spec.split(","):
        dt, *nums = item.strip().split(":")
        generic = nums[-1] == "generic"          # ...:generic also builds the tile with the chunk-wise loader
        bm, bn, bk, nw, st = (int(v) for v in (nums[:-1] if generic else nums))
        if not tile_valid(TAGS[dt][1], bm, bn, bk, nw, st):
            raise SystemExit(f"{item}: not a buildable tile")
        out.append((dt, bm, bn, bk, nw, st, generic))
    return out


def instance_list(quick=False):
    """(dtype, bm, bn, bk, nw, stages, generic) for every kernel to build."""
    out = []
    for dt, (_, es) in TAGS.items():
        bks = (32, 64) if es == 2 else (64, 128)
        for bm in (32, 64, 128, 256):
            for bn in (64, 128, 256):
                # skinny tiles (32 rows) stream B: they get one deeper K slab instead of the shallow one
                for bk in ((bks[1], 2 * bks[1]) if bm == 32 else bks):
                    for nw in (4, 8):
                        for st in (2, 3, 4):
                            if not tile_valid(es, bm, bn, bk, nw, st):
                                continue
                            if quick and not ((bm, bn) in ((256, 256), (128, 128), (64, 128)) and bk == bks[1]
                                              and st in (2, 3)):
                                continue
                            # element-wise (any stride / ragged K) variants only for two small tiles
                            generic = nw == 4 and st == 2 and bk == bks[1] and (bm, bn) in ((128, 128), (64, 128))
                            out.append((dt, bm, bn, bk, nw, st, generic))
        # 192 x 192: sixteen tiles per 3072 where the 256-wide tile has twelve -- problems whose sides are multiples of
        # 192 but leave a round of 256x256 tiles half empty (3072^3 is 144 of those on 256 CUs, and 256 of these)
        # 192 x 256 and 256 x 192 (two ring slots fit): 4096 x 2560 is 160 tiles of 256x256 and 220 / 224 of these
        if es == 2 and not quick:
            for nw in (4, 8):
                for st in (2, 3):
                    assert tile_valid(es, 192, 192, 64, nw, st)
                    out.append((dt, 192, 192, 64, nw, st, False))
                for bm, bn in ((192, 256), (256, 192)):
                    assert tile_valid(es, bm, bn, 64, nw, 2)
                    out.append((dt, bm, bn, 64, nw, 2, False))
        if es == 1 and not quick:
            for nw in (4, 8):
                for st in (2, 3):
                    assert tile_valid(es, 192, 192, 128, nw, st)
                    out.append((dt, 192, 192, 128, nw, st, False))
                for bm, bn in ((192, 256), (256, 192)):
                    assert tile_valid(es, bm, bn, 128, nw, 2)
                    out.append((dt, bm, bn, 128, nw, 2, False))
    return out


def conv_instance_list(quick=False):
    """(dtype, block_cout, block_pixels, block_k) of every conv2d forward tile to build (four waves, two LDS slots).

    The reference's own candidates (tritonix/ops/conv2d/forward.py:172-180: pixels x channels in {64, 128}^2,
    block_k in {32, 64}) and three larger tiles."""
    out = []
    for dt in ("bf16", "f16"):
        for bc, bp in ((64, 64), (64, 128), (128, 64), (128, 128), (256, 64), (256, 128), (128, 256)):
            for bk in (32, 64):
                if max(bc, bp) == 256 and bk == 32:
                    continue
                if quick and not ((bc, bp) in ((128, 128), (64, 64)) and bk == 64):
                    continue
                assert tile_valid(2, bc, bp, bk, 4, 2)
                out.append((dt, bc, bp, bk))
    return out


def parse_only_conv(spec):
    """'bf16:128:128:64,...' (dtype:block_cout:block_pixels:block_k) for development builds."""
    out = []
    for item in spec.split(","):
        dt, *nums = item.strip().split(":")
        bc, bp, bk = (int(v) for v in nums)
        if dt not in ("bf16", "f16") or not tile_valid(2, bc, bp, bk, 4, 2):
            raise SystemExit(f"{item}: not a buildable conv2d tile")
        out.append((dt, bc, bp, bk))
    return out


def write_if_changed(path, text):
    if os.path.exists(path):
        with open(path) as f:
            if f.read() == text:
                return
    with open(path, "w") as f:
        f.write(text)


def generate_conv(instances, gen):
    """Instance files of the conv2d tiles, one per (dtype, block_cout), and their table."""
    groups = {}
    for inst in instances:
        groups.setdefault((inst[0], inst[1]), []).append(inst)
    files, names = [], []
    for (dt, bc), items in sorted(groups.items()):
        name = f"conv_{dt}_c{bc}"
        tag = TAGS[dt][0]
        rows = ",\n".join(f"    TNX_CONV_ENTRY({tag}, {i[1]}, {i[2]}, {i[3]})" for i in items)
        text = (f'// generated by tritonix_amd/build.py -- do not edit\n#include "{CSRC}/conv_tile.h"\n'
                f"namespace tnx {{\nstatic ConvEntry k_{name}[] = {{\n{rows}\n}};\n"
                f"ConvGroup g_{name} = {{k_{name}, {len(items)}}};\n}}\n")
        path = os.path.join(gen, name + ".hip")
        write_if_changed(path, text)
        files.append(path)
        names.append(name)
    decl = "\n".join(f"extern ConvGroup g_{n};" for n in names)
    arr = ", ".join(f"g_{n}" for n in names)
    n = len(names)
    body = (f"  static ConvGroup all[{max(n, 1)}];\n  static bool init = false;\n"
            f"  if (!init) {{ {'ConvGroup tmp[] = {' + arr + '}; for (int i = 0; i < ' + str(n) + '; ++i) all[i] = tmp[i]; ' if n else ''}init = true; }}\n")
    text = (f'// generated by tritonix_amd/build.py -- do not edit\n#include "{CSRC}/conv_tile.h"\nnamespace tnx {{\n{decl}\n}}\n'
            f"using namespace tnx;\n"
            f'extern "C" const ConvGroup* tnx_conv_groups(int* n) {{\n{body}  *n = {n};\n  return all;\n}}\n')
    path = os.path.join(gen, "conv_groups.hip")
    write_if_changed(path, text)
    files.append(path)
    return files


def generate(instances):
    gen = os.path.join(BUILD, "gen")
    os.makedirs(gen, exist_ok=True)
    groups = {}
    for inst in instances:
        groups.setdefault((inst[0], inst[1], inst[2]), []).append(inst)
    files, names = [], []
    # at most three kernels per translation unit, the largest tiles first: the biggest unit used to take four
    # minutes on its own and set the wall time of the whole build
    parts = []
    for (dt, bm, bn), items in sorted(groups.items(), key=lambda kv: -kv[0][1] * kv[0][2]):
        for c in range(0, len(items), 3):
            suffix = f"_p{c // 3}" if len(items) > 3 else ""
            parts.append(((dt, bm, bn), f"inst_{dt}_m{bm}_n{bn}{suffix}", items[c:c + 3]))
    for (dt, bm, bn), name, items in parts:
        tag = TAGS[dt][0]
        rows = ",\n".join(
            f"    TNX_ENTRY({tag}, {i[1]}, {i[2]}, {i[3]}, {i[4]}, {i[5]}, {'true' if i[6] else 'false'})" for i in items)
        text = (f'// generated by tritonix_amd/build.py -- do not edit\n#include "{CSRC}/registry.h"\n'
                f"namespace tnx {{\nstatic KernelEntry k_{name}[] = {{\n{rows}\n}};\n"
                f"KernelGroup g_{name} = {{k_{name}, {len(items)}}};\n}}\n")
        path = os.path.join(gen, name + ".hip")
        write_if_changed(path, text)
        files.append(path)
        names.append(name)
    decl = "\n".join(f"extern KernelGroup g_{n};" for n in names)
    arr = ", ".join(f"g_{n}" for n in names)
    n = len(names)
    fill = f"KernelGroup tmp[] = {{{arr}}}; for (int i = 0; i < {n}; ++i) all[i] = tmp[i]; " if n else ""
    text = (f'// generated by tritonix_amd/build.py -- do not edit\n#include "{CSRC}/registry.h"\nnamespace tnx {{\n{decl}\n}}\n'
            f"using namespace tnx;\n"
            f'extern "C" const KernelGroup* tnx_kernel_groups(int* n) {{\n'
            f"  static KernelGroup all[{max(n, 1)}];\n  static bool init = false;\n  if (!init) {{ {fill}init = true; }}\n"
            f"  *n = {n};\n  return all;\n}}\n")
    path = os.path.join(gen, "groups.hip")
    write_if_changed(path, text)
    files.append(path)
    return files


# A compiler-generated use of M0 would collide with the DMA loader: its inline assembly writes M0 (the LDS target of
# global_load_lds) and cannot name it as clobbered.  Every device translation unit is therefore compiled with its
# assembly kept, and any mention of m0 outside an inline-assembly block fails the build.
_M0 = re.compile(r"(?<![\w.$])m0(?![\w])")
_REMARK = re.compile(r"remark: .*?:\d+:\d+:\s+(Function Name|TotalSGPRs|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|"
                     r"SGPRs Spill|VGPRs Spill|LDS Size \[bytes/block\]): (\S+)")


def compiler_m0_uses(asm_path):
    """(line number, text) of every instruction outside inline assembly that names M0."""
    found, inside = [], False
    with open(asm_path, errors="replace") as f:
        for n, line in enumerate(f, 1):
            if ";;#ASMSTART" in line:
                inside = True
            elif ";;#ASMEND" in line:
                inside = False
            elif not inside and _M0.search(line.split(";", 1)[0]):
                found.append((n, line.strip()))
    return found


def parse_resources(stderr):
    """{mangled kernel name: {"sgpr", "vgpr", "agpr", "scratch", "occupancy", "sgpr_spill", "vgpr_spill", "lds"}} from the
    compiler's -Rpass-analysis=kernel-resource-usage remarks (no disassembly involved)."""
    names = {"TotalSGPRs": "sgpr", "VGPRs": "vgpr", "AGPRs": "agpr", "ScratchSize [bytes/lane]": "scratch",
             "Occupancy [waves/SIMD]": "occupancy", "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill",
             "LDS Size [bytes/block]": "lds"}
    out, cur = {}, None
    for m in _REMARK.finditer(stderr):
        key, val = m.group(1), m.group(2)
        if key == "Function Name":
            cur = out.setdefault(val, {})
        elif cur is not None:
            cur[names[key]] = int(val)
    return out


_resources = {}


def _compile(src, obj, verbose, force=True):
    deps = [src, os.path.join(CSRC, "gemm_tile.h"), os.path.join(CSRC, "gemm_skinny.h"), os.path.join(CSRC, "registry.h"),
            os.path.join(CSRC, "conv_tile.h"),
            os.path.join(ROOT, "include", "tritonix_hip.h"), os.path.abspath(__file__)]
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(d) for d in deps):
        return obj
    t0 = time.time()
    cmd = [HIPCC, *DEVICE_FLAGS, "-save-temps=obj", "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
    _resources.update(parse_resources(r.stderr))
    stem = obj[:-2]
    asm = f"{stem}-hip-amdgcn-amd-amdhsa-{ARCH}.s"
    uses = compiler_m0_uses(asm)
    for tmp in glob.glob(glob.escape(stem) + "-hip-amdgcn-*") + glob.glob(glob.escape(stem) + "-host-*") + glob.glob(glob.escape(stem) + ".hip-hip-*"):
        os.remove(tmp)
    if uses:
        raise RuntimeError(f"{src}: the compiler generated {len(uses)} use(s) of M0 outside inline assembly, e.g. line "
                           f"{uses[0][0]}: {uses[0][1]} -- the DMA loader's inline assembly owns M0 (gemm_tile.h: dma16)")
    if verbose:
        print(f"  [{time.time() - t0:5.1f}s] {os.path.basename(src)}", flush=True)
    return obj


def demangled_tile(name):
    """'bf16 256x256x64 w4 s2 fast' from a mangled gemm_tile_kernel instantiation (None for other kernels)."""
    m = re.search(r"gemm_tile_kernelINS_(\d)Tag(\w+?)ENS_7TileCfgIS1_Li(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)EEELb(\d)ELb(\d)ELb(\d)ELb(\d)E", name)
    if not m:
        return None
    _, tag, bm, bn, bk, nw, st, fast, persist, bt, conv = m.groups()
    kind = "conv" if conv == "1" else "bt" if bt == "1" else "persistent" if persist == "1" else "fast" if fast == "1" else "generic"
    return f"{tag.lower()} {bm}x{bn}x{bk} w{nw} s{st} {kind}"


def build(jobs=None, quick=False, verbose=True, force=True, only=None, out=None, defines=(), only_conv=None):
    """Compile every kernel for gfx950 and link the shared library.

    ``only`` / ``out`` / ``defines`` are for development builds: a few tiles, linked to another path, with extra
    ``-D`` macros; they use their own object directory so the full build's objects stay valid."""
    global BUILD
    jobs = jobs or min(8, os.cpu_count() or 1)
    instances = parse_only(only) if only else ([] if only_conv else instance_list(quick=quick))
    conv_instances = parse_only_conv(only_conv) if only_conv else ([] if only else conv_instance_list(quick=quick))
    lib = out or LIB
    if only or only_conv or out or defines:
        BUILD = os.path.join(ROOT, "build", "dev_" + os.path.basename(lib).replace(".", "_"))
    DEVICE_FLAGS.extend(f"-D{d}" for d in defines)
    srcs = generate(instances) + generate_conv(conv_instances, os.path.join(BUILD, "gen")) + [
        os.path.join(CSRC, "capi.hip"), os.path.join(CSRC, "skinny.hip"),
        os.path.join(CSRC, "conv.hip")]
    objdir = os.path.join(BUILD, "obj")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    if verbose:
        print(f"building {len(instances)} GEMM and {len(conv_instances)} conv2d tile kernels in {len(srcs)} translation units, "
              f"{jobs} jobs", flush=True)
    t0 = time.time()
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile(so[0], so[1], verbose, force), zip(srcs, objs)))
    # stale objects of groups that no longer exist must not be linked
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", lib + ".tmp", *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    os.replace(lib + ".tmp", lib)
    # registers, scratch and LDS of every kernel compiled in this run, as the compiler reported them
    table = {demangled_tile(k) or k: v for k, v in _resources.items()}
    with open(os.path.join(BUILD, "kernel_resources.json"), "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
    if verbose:
        print(f"linked {lib} in {time.time() - t0:.1f}s; no compiler-generated use of M0; "
              f"kernel resources in {os.path.join(BUILD, 'kernel_resources.json')}", flush=True)
    return lib


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--quick", action="store_true", help="build a small subset of the tile kernels (development)")
    ap.add_argument("--incremental", action="store_true", help="development: keep objects that are newer than their sources")
    ap.add_argument("--only", default=None, help="development: build just these tiles, dtype:bm:bn:bk:warps:stages,...")
    ap.add_argument("--only-conv", default=None, help="development: build just these conv2d tiles, dtype:cout:pixels:bk,...")
    ap.add_argument("--out", default=None, help="development: link to this path instead of the package's library")
    ap.add_argument("-D", dest="defines", action="append", default=[], help="development: extra macro for the device code")
    args = ap.parse_args(argv)
    build(jobs=args.jobs, quick=args.quick, only=args.only, out=args.out, defines=args.defines, force=not args.incremental,
          only_conv=args.only_conv)
    return 0


if __name__ == "__main__":
    sys.exit(main())
