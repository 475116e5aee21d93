"""Builds libguffin_hip.so (gfx950 only) from guffin_amd/csrc with hipcc, and the same device code once more as
plain code objects (guffin_amd/hsaco/*.hsaco with kernargs.txt) for the chain engine, which loads kernels through
the HSA runtime and writes their dispatch packets itself."""
import concurrent.futures
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
HSACO = os.path.join(HERE, "hsaco")
LIB = os.path.join(HERE, "libguffin_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
READELF = os.environ.get("LLVM_READELF", "/opt/rocm/llvm/bin/llvm-readelf")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]

# offsets of the implicit kernel arguments inside their block (code object v5)
HIDDEN = {
    "hidden_block_count_x": 0, "hidden_block_count_y": 4, "hidden_block_count_z": 8,
    "hidden_group_size_x": 12, "hidden_group_size_y": 14, "hidden_group_size_z": 16,
    "hidden_remainder_x": 18, "hidden_remainder_y": 20, "hidden_remainder_z": 22,
    "hidden_global_offset_x": 40, "hidden_global_offset_y": 48, "hidden_global_offset_z": 56,
    "hidden_grid_dims": 64, "hidden_dynamic_lds_size": 120,
}


def _compile(src):
    obj = os.path.join(OBJ, os.path.splitext(os.path.basename(src))[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
    return obj, r.stderr


def _code_object(src):
    out = os.path.join(HSACO, os.path.splitext(os.path.basename(src))[0] + ".hsaco")
    cmd = [HIPCC, *FLAGS, "--cuda-device-only", "--no-gpu-bundle-output", src, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc (device only) failed for %s:\n%s" % (src, r.stderr))
    return out


def kernarg_rows(code_object):
    """(kernel name, end of the explicit arguments, start of the implicit block or -1) for every kernel of a code
    object, from its metadata note.  Raises on an implicit argument the chain engine does not fill."""
    import yaml
    text = subprocess.run([READELF, "--notes", code_object], capture_output=True, text=True, check=True).stdout
    rows = []
    start = text.find("---")
    end = text.find("\n...", start)
    if start < 0 or end < 0:
        return rows
    meta = yaml.safe_load(text[start + 3:end])
    for k in meta.get("amdhsa.kernels", []):
        explicit_end, hidden_start = 0, -1
        for a in k.get(".args", []):
            kind = a[".value_kind"]
            if kind.startswith("hidden_"):
                if kind not in HIDDEN:
                    raise RuntimeError("%s uses %s, which the chain engine does not provide" % (k[".name"], kind))
                base = a[".offset"] - HIDDEN[kind]
                if hidden_start >= 0 and base != hidden_start:
                    raise RuntimeError("%s: implicit arguments are not laid out as expected" % k[".name"])
                hidden_start = base
            else:
                explicit_end = max(explicit_end, a[".offset"] + a[".size"])
        if hidden_start >= 0 and hidden_start != (explicit_end + 7) // 8 * 8:
            raise RuntimeError("%s: the implicit block does not follow the explicit arguments" % k[".name"])
        rows.append((k[".name"], explicit_end, hidden_start))
    return rows


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(HSACO, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))  # .cpp: host only
    device_sources = [s for s in sources if s.endswith(".hip")]
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        objects = pool.map(_compile, sources)
        code_objects = pool.map(_code_object, device_sources)
        results = list(objects)
        code_objects = list(code_objects)
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            lines = [l for l in err.splitlines() if "packed-fp32-ops" not in l and l.strip()]
            if lines:
                print("\n".join(lines))
    with open(os.path.join(HSACO, "kernargs.txt"), "w") as table:
        for co in code_objects:
            for name, explicit_end, hidden_start in kernarg_rows(co):
                table.write("%s %d %d\n" % (name, explicit_end, hidden_start))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs,
                        "-L/opt/rocm/lib", "-lhsa-runtime64", "-ldl"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
