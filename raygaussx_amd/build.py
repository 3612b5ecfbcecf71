"""Compiles librgx.so (HIP, gfx950) in-tree with hipcc.

``python -m raygaussx_amd.build`` or ``build()``.  The flags matter:
``-ffp-contract=off`` keeps the hit predicate's arithmetic identical to a CPU
evaluation (fused multiply-adds only where the source says fmaf);
``-munsafe-fp-atomics`` selects the hardware fp32 atomic add for the gradient
scatter; packed-fp32 code generation is disabled; the march kernels' source is compiled without
machine-code loop-invariant code motion, in two pieces with different scheduling (``UNITS``).

``python -m raygaussx_amd.build --resources`` also prints what every kernel takes: registers,
bytes of register spills per lane, LDS.  The march kernels are sized for three wavefronts per SIMD
(168 registers) and twelve tiles per CU (12 800 bytes of LDS); a change that pushes spills into
their sweep loops costs more than most optimisations gain, so look at this table after touching
them.

``python -m raygaussx_amd.build --sections`` builds ``librgx_sections.so``, a diagnostic copy whose march
kernels count the cycles each of their sections takes (see ``bench.py --sections``).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librgx.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
         "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]
# The march kernels have no register to spare, and what the machine-code loop-invariant code motion hoists out
# of their slab loops (addresses, constants, selects of wave-uniform values) it pays for with spills inside them:
# without it the recording forward runs 3-4 % faster (36 -> 20 bytes of spills per lane; the plain forward and
# the replaying backward lose theirs altogether and run as before).
NO_LICM = ["-mllvm", "-disable-machine-licm=1"]
# The march source is compiled twice: once for everything but the backward kernels, without the scheduling pass
# that runs after register allocation (the forward without a record runs 1-3 % faster on what the first
# scheduler left), and once for the backward kernels alone, which that pass helps by about 1 %.
# (source, object name, flags of that compilation)
UNITS = [("rgx_api.hip", "rgx_api", []), ("rgx_build.hip", "rgx_build", []), ("rgx_pergauss.hip", "rgx_pergauss", []),
         ("rgx_image.hip", "rgx_image", []),
         ("rgx_march.hip", "rgx_march", ["-DRGX_MARCH_TU=1", *NO_LICM, "-mllvm", "-enable-post-misched=0"]),
         ("rgx_march.hip", "rgx_march_bwd", ["-DRGX_MARCH_TU=2", *NO_LICM])]
# The diagnostic build keeps the march source in one piece (its cycle table is one device variable).
UNITS_SECTIONS = UNITS[:4] + [("rgx_march.hip", "rgx_march", NO_LICM)]


def _resource_table(compiler_output):
    """Kernel name, VGPRs, spill bytes per lane, waves per SIMD, LDS bytes from -Rpass-analysis remarks."""
    rows, cur = [], None
    for line in compiler_output.splitlines():
        if "remark:" not in line:
            continue
        text = line.split("remark:", 1)[1].strip()
        key, _, val = text.partition(":")
        val = val.split("[")[0].strip()
        if key.strip() == "Function Name":
            cur = {"name": val}
            rows.append(cur)
        elif cur is not None and key.strip() in ("VGPRs", "ScratchSize [bytes/lane]", "Occupancy [waves/SIMD]", "LDS Size [bytes/block]"):
            cur[key.strip()] = val
    seen, out = set(), []
    for r in rows:     # the host pass repeats the device pass's remarks
        if r["name"] in seen or "VGPRs" not in r:
            continue
        seen.add(r["name"])
        out.append(f"{r['name'][:70]:70s} vgpr {r.get('VGPRs', '?'):>4s}  spill B/lane {r.get('ScratchSize [bytes/lane]', '?'):>4s}  "
                   f"waves/SIMD {r.get('Occupancy [waves/SIMD]', '?'):>2s}  LDS {r.get('LDS Size [bytes/block]', '?'):>6s}")
    return "\n".join(out)


def build(verbose=False, extra=(), lib=LIB, tag="", resources=False, units=None):
    """``extra``: more hipcc flags; ``lib`` / ``tag``: write a differently named library and objects;
    ``resources``: print every kernel's register, spill and LDS use; ``units``: the compilations (``UNITS``)."""
    objs = []
    procs = []
    if resources:
        extra = [*extra, "-Rpass-analysis=kernel-resource-usage"]
    for src, name, flags in (UNITS if units is None else units):
        obj = os.path.join(CSRC, name + tag + ".o")
        cmd = ["hipcc", *FLAGS, *flags, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((name, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(out, file=sys.stderr)
        elif resources:
            print(f"-- {src}\n{_resource_table(out)}", flush=True)
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib]
    subprocess.check_call(cmd)
    return lib


SECTIONS_LIB = os.path.join(HERE, "librgx_sections.so")


def build_sections(**kw):
    """The diagnostic build with the per-section cycle census of the march kernels compiled in
    (``-DRGX_SECTION_CLOCKS``): ``librgx_sections.so`` beside the product library, which it never replaces.
    ``RGX_LIB_PATH=raygaussx_amd/librgx_sections.so python bench.py --sections`` reads the census."""
    return build(extra=["-DRGX_SECTION_CLOCKS"], lib=SECTIONS_LIB, tag="_sections", units=UNITS_SECTIONS, **kw)


if __name__ == "__main__":
    if "--sections" in sys.argv[1:]:
        print(build_sections(verbose=True, resources="--resources" in sys.argv[1:]))
    else:
        print(build(verbose=True, resources="--resources" in sys.argv[1:]))
