"""In-tree build of the kukeon_amd HIP extension for gfx950.

Drives hipcc directly (native .hip sources — no hipify, no CUDA paths) and
links against libtorch so the resulting ``_C.so`` lives inside the package
tree and travels with repo snapshots.  Cross-compiles fine on a GPU-less box.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent.parent  # kukeon_amd/
CSRC = PKG_DIR / "ops" / "csrc"
OBJ_DIR = PKG_DIR / "ops" / "_build"
SO_PATH = PKG_DIR / "_C.so"
ARCH = os.environ.get("KUKEON_GFX_ARCH", "gfx950")

# Kernel groups: each links into its own module, so a model that needs one
# group does not wait for the others to compile.
#   core -> kukeon_amd/_C.so      (Llama/Mixtral op set, sampler, GEMMs)
#   mix  -> kukeon_amd/_C_mix.so  (fp32-residual norm, clamped GLU, short
#                                  convolution + rotary, differential attention)
MIX_SOURCES = [
    "resid_norm.hip",
    "glu_clamp.hip",
    "short_conv.hip",
    "diff_attn.hip",
    "diff_attn_mfma.hip",
    "diff_attn_decode.hip",
    "bindings_mix.cpp",
]

#   recur -> kukeon_amd/_C_recur.so (sandwich norms, convolution with
#                                  activation, state-space scan, latent
#                                  attention, table-routed experts)
RECUR_SOURCES = [
    "resid_norm.hip",
    "short_conv.hip",
    "conv_act.hip",
    "ssm_scan.hip",
    "recur_elem.hip",
    "latent_attn.hip",
    "table_moe.hip",
    "bindings_recur.cpp",
]

#   hyb -> kukeon_amd/_C_hyb.so   (output-side layer norm, chunk-local
#                                  attention, decayed linear attention, gated
#                                  activations, routed experts, latent
#                                  attention)
HYB_SOURCES = [
    "layer_norm.hip",
    "glu_clamp.hip",
    "chunk_attn.hip",
    "prefill_attn.hip",
    "lightning.hip",
    "routed_moe.hip",
    "latent_attn.hip",
    "recur_elem.hip",
    "table_moe.hip",
    "bindings_hyb.cpp",
]

#   strm -> kukeon_amd/_C_strm.so (several residual streams, token shift,
#                                  linear attention with a token-dependent
#                                  decay, windowed attention over key-only
#                                  pages, group-limited routing)
STRM_SOURCES = [
    "stream_mix.hip",
    "decay_scan.hip",
    "window_attn.hip",
    "short_conv.hip",
    "chunk_attn.hip",
    "prefill_attn.hip",
    "routed_moe.hip",
    "glu_clamp.hip",
    "table_moe.hip",
    "bindings_strm.cpp",
]

SOURCES = [
    "rmsnorm.hip",
    "activation.hip",
    "rope_kv.hip",
    "paged_attn.hip",
    "prefill_attn.hip",
    "sampling.hip",
    "moe.hip",
    "skinny_gemm.hip",
    "bindings.cpp",
]


def _torch_paths():
    from torch.utils import cpp_extension

    return cpp_extension.include_paths(), cpp_extension.library_paths()


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n")
        sys.stderr.write(proc.stdout[-4000:] + "\n" + proc.stderr[-8000:] + "\n")
        raise RuntimeError(f"build command failed (rc={proc.returncode})")


GROUPS = {
    "core": ("_C", SOURCES),
    "mix": ("_C_mix", MIX_SOURCES),
    "recur": ("_C_recur", RECUR_SOURCES),
    "hyb": ("_C_hyb", HYB_SOURCES),
    "strm": ("_C_strm", STRM_SOURCES),
}


def so_path(group: str) -> Path:
    return PKG_DIR / (GROUPS[group][0] + ".so")


def build(verbose: bool = True, force: bool = False,
          groups=None) -> Path:
    """Compile and link the given kernel groups (default: all)."""
    out = None
    done: set = set()       # sources compiled in this call (groups share some)
    for g in (groups or list(GROUPS)):
        out = _build_group(g, verbose, force, done)
    return out


def _build_group(group: str, verbose: bool, force: bool,
                 done: set = None) -> Path:
    modname, sources = GROUPS[group]
    SO_PATH = so_path(group)
    inc, libdirs = _torch_paths()
    py_inc = sysconfig.get_paths()["include"]
    OBJ_DIR.mkdir(parents=True, exist_ok=True)

    common_flags = [
        f"--offload-arch={ARCH}",
        "-O3",
        "-std=c++17",
        "-fPIC",
        "-DNDEBUG",
        "-D__HIP_NO_HALF_OPERATORS__=1",
        "-D__HIP_NO_HALF_CONVERSIONS__=1",
        f"-DTORCH_EXTENSION_NAME={modname}",
        # packed fp32 VALU forms are kept out of all device code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-DUSE_ROCM=1",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-D_GLIBCXX_USE_CXX11_ABI=1",
        "-fno-gpu-rdc",
        "-Wno-unused-result",
    ]
    common_flags += [f"-I{p}" for p in inc]
    common_flags += [f"-I{py_inc}", f"-I{CSRC}"]

    hdr_mtime = max(p.stat().st_mtime for p in CSRC.glob("*.h"))
    objs = []
    todo = []
    for src in sources:
        sp = CSRC / src
        op = OBJ_DIR / (src.rsplit(".", 1)[0] + ".o")
        objs.append(op)
        if ((not force or (done is not None and src in done))
                and op.exists()
                and op.stat().st_mtime > max(sp.stat().st_mtime, hdr_mtime)):
            continue
        if done is not None:
            done.add(src)
        cmd = ["hipcc", "-c", str(sp), "-o", str(op)] + common_flags
        if src.endswith(".cpp"):
            cmd.append("-x")
            cmd.append("c++")
        todo.append((src, cmd))

    def _one(item):
        if verbose:
            print(f"[kukeon_amd.build] hipcc -c {item[0]}", flush=True)
        _run(item[1])

    if todo:
        from concurrent.futures import ThreadPoolExecutor
        jobs = max(1, min(len(todo), int(os.environ.get("MAX_JOBS", "0") or 0)
                          or (os.cpu_count() or 4), 16))
        with ThreadPoolExecutor(jobs) as pool:
            list(pool.map(_one, todo))

    if force or not SO_PATH.exists() or any(
            o.stat().st_mtime > SO_PATH.stat().st_mtime for o in objs):
        if verbose:
            print(f"[kukeon_amd.build] linking {SO_PATH.name}")
        link = (
            ["hipcc", "-shared", "-fPIC", "-o", str(SO_PATH)]
            + [str(o) for o in objs]
            + [f"-L{d}" for d in libdirs]
            + [
                "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
                "-ltorch_python", "-lamdhip64",
            ]
            + [f"-Wl,-rpath,{d}" for d in libdirs]
        )
        _run(link)
    return SO_PATH


if __name__ == "__main__":
    names = [a for a in sys.argv[1:] if not a.startswith("-")]
    build(force="--force" in sys.argv, groups=names or None)
    for g in (names or list(GROUPS)):
        print(f"built {so_path(g)}")
