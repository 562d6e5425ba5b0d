"""Builds libtrident_attn.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

    python -m trident_amd.build               # compile every csrc/*.hip and link
    python -m trident_amd.build --resources   # also print the per-kernel register / LDS / scratch table

Every build reads the compiler's kernel-resource-usage remarks and FAILS when any kernel of the library uses scratch
memory (spilled vector registers): a scratch reload is a vector-memory load, and the kernels' hand-counted vmcnt waits
would then drain the tile prefetch on every reload. It also fails when a kernel of the five benchmark configurations is
missing from the build.
"""
import concurrent.futures
import glob
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT = os.path.join(HERE, "libtrident_attn.so")
PROBE_SRC = os.path.join(HERE, "probe", "probe.hip")   # calibration kernels: a library of their own (include/tri_probe.h)
PROBE_OUT = os.path.join(HERE, "libtri_probe.so")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-pass-failed",  # 4-wave variants ask for two workgroups per CU and get one (LDS): known, not an error
    "-Wno-inline-asm",  # the LDS-direct load helpers name M0 as clobbered, which clang reports as a reserved register
    "-I", INCLUDE,
    "-I", CSRC,
    "-Rpass-analysis=kernel-resource-usage",
]

# The kernels the five benchmark configurations launch (demangled name without the parameter list).
BASELINE_KERNELS = {
    "mfma_fwd_kernel<_Float16, 64, 8, false, 0, false, false>": "C2 fwd",
    "mfma_fwd_kernel<__bf16, 128, 8, true, 0, false, false>": "C3 fwd",
    "mfma_dq_phased_kernel<__bf16, 128, true, false, true>": "C3 dQ + delta",
    "mfma_dkdv_phased_kernel<__bf16, 128, true, false, 0>": "C3 dK/dV",
    "mfma_fwd_kernel<__bf16, 64, 8, false, 1, false, false>": "C4 fwd",
    "delta_kernel<__bf16, 64>": "C4 delta",
    "mfma_dkdv_wide_kernel<__bf16, 64, 8, false, 1, false, false>": "C4 dK/dV",
    "mfma_dq_kernel<__bf16, 64, 8, false, 1, false, false, false, false>": "C4 dQ",
    "mfma_fwd_kernel<__bf16, 128, 8, true, 0, true, false>": "C5 fwd",
    "mfma_dq_phased_kernel<__bf16, 128, true, true, true>": "C5 dQ + delta",
    "mfma_dkdv_phased_kernel<__bf16, 128, true, true, 0>": "C5 dK/dV",
    "mfma32_fwd_kernel<float, 32>": "C1 fwd",
}
_FIELDS = [("TotalSGPRs", "sgpr"), ("VGPRs", "vgpr"), ("AGPRs", "agpr"), ("ScratchSize [bytes/lane]", "scratch"),
           ("Occupancy [waves/SIMD]", "occupancy"), ("SGPRs Spill", "sgpr_spill"), ("VGPRs Spill", "vgpr_spill"),
           ("LDS Size [bytes/block]", "lds")]


def _parse_resources(stderr):
    """{mangled kernel name: {field: int}} from the -Rpass-analysis=kernel-resource-usage remarks."""
    out, cur = {}, None
    for line in stderr.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        if cur is None:
            continue
        for label, key in _FIELDS:
            m = re.search(r"remark:\s+" + re.escape(label) + r": (\d+)", line)
            if m:
                cur[key] = int(m.group(1))
    return out


def _demangle(names):
    """Readable names of this library's kernels (tri::(anonymous)::name<type / int / bool arguments>(...))."""
    out = {}
    for n in names:
        m = re.match(r"_ZN3tri12_GLOBAL__N_1(\d+)", n)
        if not m:
            out[n] = n
            continue
        ln = int(m.group(1))
        name, rest = n[m.end():m.end() + ln], n[m.end() + ln:]
        args = []
        if rest.startswith("I"):
            rest = rest[1:]
            while rest and not rest.startswith("E"):
                for pat, fn in ((r"DF16_", lambda g: "_Float16"), (r"DF16b", lambda g: "__bf16"), (r"f", lambda g: "float"),
                                (r"Li(\d+)E", lambda g: g.group(1)), (r"Lb([01])E", lambda g: "true" if g.group(1) == "1" else "false")):
                    g = re.match(pat, rest)
                    if g:
                        args.append(fn(g))
                        rest = rest[g.end():]
                        break
                else:
                    args, rest = ["?"], ""
        out[n] = name + ("<" + ", ".join(args) + ">" if args else "")
    return out


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    lines, skip = [], 0
    for l in res.stderr.splitlines():  # (a remark is followed by two lines quoting the source)
        if "packed-fp32-ops" in l:
            continue
        if "-Rpass-analysis=kernel-resource-usage" in l:
            skip = 2
            continue
        if skip and (re.match(r"\s*\d+ \|", l) or re.match(r"\s*\|", l)):
            skip -= 1
            continue
        skip = 0
        lines.append(l)
    err = "\n".join(lines)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj, _parse_resources(res.stderr)


def resource_table(resources):
    names = _demangle(sorted(resources))
    rows = sorted(((names[m], r) for m, r in resources.items()), key=lambda x: x[0])
    head = f"{'kernel':<64} {'config':<14} {'VGPR':>5} {'AGPR':>5} {'SGPR':>5} {'SGPR spill':>10} {'VGPR spill':>10} " \
           f"{'scratch B':>9} {'LDS B':>7} {'waves/SIMD':>10}"
    out = [head]
    for name, r in rows:
        out.append(f"{name:<64} {BASELINE_KERNELS.get(name, ''):<14} {r.get('vgpr', 0):>5} {r.get('agpr', 0):>5} "
                   f"{r.get('sgpr', 0):>5} {r.get('sgpr_spill', 0):>10} {r.get('vgpr_spill', 0):>10} {r.get('scratch', 0):>9} "
                   f"{r.get('lds', 0):>7} {r.get('occupancy', 0):>10}")
    return "\n".join(out)


def check_baseline_kernels(resources):
    names = _demangle(sorted(resources))
    found = {names[m]: r for m, r in resources.items()}
    missing = [k for k in BASELINE_KERNELS if k not in found]
    if missing:
        raise RuntimeError("kernels of the benchmark configurations not found in the build: " + ", ".join(missing))
    bad = [f"{k}{' (' + BASELINE_KERNELS[k] + ')' if k in BASELINE_KERNELS else ''}: {r.get('scratch', 0)} bytes of scratch per lane"
           for k, r in sorted(found.items()) if r.get("scratch", 0) > 0]
    if bad:
        raise RuntimeError("kernels spill vector registers to scratch:\n  " + "\n  ".join(bad))


def build(verbose=True, resources=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources) + 1)) as pool:
        results = list(pool.map(_compile, sources + [PROBE_SRC]))
    probe_obj = results.pop()[0]
    objs = [o for o, _ in results]
    usage = {}
    for _, r in results:
        usage.update(r)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    subprocess.check_call(cmd)
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_OUT, probe_obj])
    if resources:
        print(resource_table(usage))
    check_baseline_kernels(usage)
    if verbose:
        print(f"built {OUT} from {len(sources)} sources; {len(usage)} kernels, none uses scratch")
    return OUT


if __name__ == "__main__":
    build(resources="--resources" in sys.argv[1:])
