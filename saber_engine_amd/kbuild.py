"""Build step of the gfx950 plugin set: the counterpart of the reference's `saber-kbuild`
(crates/saber-kernels/src/bin/saber-kbuild.rs:186-251) and its source ladder
(crates/saber-kernels/src/ladder.rs:12-36).

For every kernel stem: resolve `<k>.gfx950.hip -> <k>.gfx95.hip -> <k>.hip`, compile with
`hipcc --genco --offload-arch=gfx950 -O3 ...`, hash sha256(preprocessed source ++ flags), and
write `prebuilt/gfx950/<k>.hsaco` + `<k>.manifest.toml` (schema 1, every number read back from
the code object that was just built). Also builds the host library `libsaber_iu8.so`, the
test-only tap object under `prebuilt/gfx950/taps/`, and writes the launch law as data to
`prebuilt/gfx950/macaq_iu8.band.toml`.

    python -m saber_engine_amd.kbuild            # everything
    python -m saber_engine_amd.kbuild macaq_iu8  # one plugin
"""
import ctypes
import glob
import hashlib
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
KERNELS = os.path.join(PKG, "csrc", "kernels")
HOST = os.path.join(PKG, "csrc", "host")
ARCH = "gfx950"
PREBUILT = os.path.join(ROOT, "prebuilt", ARCH)
LIB = os.path.join(PKG, "libsaber_iu8.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: every product and sum rounds where the source says (the epilogue contract);
# the packed-fp32 feature is switched off for every device compile of this tree.
FLAGS = f"--genco --offload-arch={ARCH} -O3 -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops"
PLUGINS = ("macaq_iu8", "macaq_iu8f", "macaq_i8q", "mxfp4_hadi8", "attn_glue_hadi8", "moe_iu8", "iu8_probe")
# test infrastructure (accumulator and table taps of the parity suite): built beside the plugin
# directory, where opening the plugin set does not see it
TAPS = ("iu8_taps",)
TAPS_DIR = os.path.join(PREBUILT, "taps")
BAND = os.path.join(PREBUILT, "macaq_iu8.band.toml")
DEVICE_PROFILE = os.path.join(PREBUILT, "device_profile.toml")


def candidates(stem, arch):
    """Most specific first: gfx950 -> k.gfx950.hip, k.gfx95.hip, k.hip."""
    out = [f"{stem}.{arch}.hip"]
    digits = arch[3:] if arch.startswith("gfx") else ""
    if len(digits) > 2:
        fam = "gfx" + digits[:2]
        if fam != arch:
            out.append(f"{stem}.{fam}.hip")
    out.append(f"{stem}.hip")
    return out


def resolve_source(stem, arch=ARCH, directory=KERNELS):
    for c in candidates(stem, arch):
        p = os.path.join(directory, c)
        if os.path.isfile(p):
            return p
    return None


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + r.stderr)
    return r


def build_lib():
    """Host sources as plain C++; the one file with device code (the static workspace array and its
    fill kernel) as HIP for gfx950, its fat binary linked into the library."""
    inc = "-I" + os.path.join(ROOT, "include")
    objs = []
    odir = os.path.join(PKG, "build")
    os.makedirs(odir, exist_ok=True)
    for src in sorted(glob.glob(os.path.join(HOST, "*.cpp"))):
        obj = os.path.join(odir, os.path.basename(src) + ".o")
        _run([HIPCC, "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", inc, "-c", src, "-o", obj])
        objs.append(obj)
    for src in sorted(glob.glob(os.path.join(HOST, "*.hip"))):
        obj = os.path.join(odir, os.path.basename(src) + ".o")
        _run([HIPCC, "-x", "hip", f"--offload-arch={ARCH}", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Xclang", "-target-feature", "-Xclang",
              "-packed-fp32-ops", inc, "-c", src, "-o", obj])
        objs.append(obj)
    _run([HIPCC, "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def _lib():
    L = ctypes.CDLL(LIB)
    L.saber_iu8_last_error.restype = ctypes.c_char_p
    return L


def build_plugin(stem, out_dir=PREBUILT):
    src = resolve_source(stem)
    if src is None:
        raise FileNotFoundError(f"no source for `{stem}` under {KERNELS}")
    os.makedirs(out_dir, exist_ok=True)
    flags = FLAGS.split()
    pp = _run([HIPCC] + flags + ["-E", "-P", src, "-o", "-"]).stdout.encode()
    build_hash = hashlib.sha256(pp + FLAGS.encode()).hexdigest()
    hsaco = os.path.join(out_dir, f"{stem}.hsaco")
    _run([HIPCC] + flags + [src, "-o", hsaco])
    with open(src, "rb") as f:
        src_sha = hashlib.sha256(f.read()).hexdigest()
    manifest = os.path.join(out_dir, f"{stem}.manifest.toml")
    L = _lib()
    rc = L.saber_iu8_manifest_write(hsaco.encode(), stem.encode(), ARCH.encode(), os.path.relpath(src, ROOT).encode(),
                                    src_sha.encode(), FLAGS.encode(), build_hash.encode(), manifest.encode())
    if rc != 0:
        raise RuntimeError(f"manifest for {stem}: {L.saber_iu8_last_error().decode()}")
    refusal = ctypes.c_int(0)
    rc = L.saber_iu8_manifest_validate(manifest.encode(), ARCH.encode(), ctypes.byref(refusal))
    if rc != 0:
        raise RuntimeError(f"{stem}: the fresh manifest does not validate: {L.saber_iu8_last_error().decode()}")
    return hsaco, manifest


def _text_of(entry):
    L = _lib()
    fn = getattr(L, entry)
    need = ctypes.c_size_t(0)
    fn(None, ctypes.c_size_t(0), ctypes.byref(need))
    buf = ctypes.create_string_buffer(need.value)
    if fn(buf, ctypes.c_size_t(need.value), None) != 0:
        raise RuntimeError(entry + ": " + L.saber_iu8_last_error().decode())
    return buf.value.decode()


def band_text():
    """The launch law as TOML text, straight from the host library."""
    return _text_of("saber_iu8_band_toml")


def device_profile_text():
    """The target's DeviceProfile as TOML text, straight from the host library."""
    return _text_of("saber_iu8_device_profile_toml")


def write_band(path=BAND):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(band_text())
    with open(DEVICE_PROFILE, "w") as f:
        f.write(device_profile_text())
    return path


def build_all(stems=None):
    build_lib()
    built = []
    for stem in stems or PLUGINS + TAPS:
        if resolve_source(stem) is None:
            continue
        built.append(build_plugin(stem, TAPS_DIR if stem in TAPS else PREBUILT))
    if not stems:
        write_band()
    return built


if __name__ == "__main__":
    for h, m in build_all(sys.argv[1:] or None):
        print("built", os.path.relpath(h, ROOT), os.path.relpath(m, ROOT))
