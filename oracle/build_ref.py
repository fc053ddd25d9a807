"""Compile the reference's own C++ search kernels, in place, into oracle/_ref/.

TEST INFRASTRUCTURE ONLY.  The sources are read where they lie under the reference
tree (kernels/cpp/torch_ext{,_v2,_v3,_v4}.cpp); nothing is copied into this
repository and only the built extension modules land in oracle/_ref/ (git-ignored).
The flags are the reference's own (kernels/cpp/torch_ext_loader.py:37-59) except
that -march=native becomes -march=x86-64-v3, so that a module built on one host
also runs on a host with a different CPU.

    python oracle/build_ref.py [--reference /root/reference]
"""
from __future__ import annotations

import argparse
import importlib.util
import os
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
REF_DIR = HERE / "_ref"

# module name -> source file under <reference>/kernels/cpp/
REF_SOURCES = {
    "hira_ref_v1": "torch_ext.cpp",
    "hira_ref_v2": "torch_ext_v2.cpp",
    "hira_ref_v3": "torch_ext_v3.cpp",
    "hira_ref_v4": "torch_ext_v4.cpp",
}
CFLAGS = ["-O3", "-march=x86-64-v3", "-ffast-math", "-fopenmp"]


def build(reference: str = "/root/reference", verbose: bool = False) -> list[str]:
    """Build every reference extension whose source exists; returns the module names."""
    from torch.utils.cpp_extension import load

    src_dir = Path(reference) / "kernels" / "cpp"
    built = []
    for name, fname in REF_SOURCES.items():
        src = src_dir / fname
        if not src.exists():
            continue
        out_dir = REF_DIR / name
        out_dir.mkdir(parents=True, exist_ok=True)
        load(
            name=name,
            sources=[str(src)],
            extra_cflags=CFLAGS,
            extra_ldflags=["-fopenmp"],
            build_directory=str(out_dir),
            verbose=verbose,
        )
        built.append(name)
    return built


def load_ref(name: str = "hira_ref_v3"):
    """Import a previously built reference extension from oracle/_ref/, or return None."""
    so = REF_DIR / name / f"{name}.so"
    if not so.exists():
        return None
    import torch  # noqa: F401  (the extension links against libtorch)

    spec = importlib.util.spec_from_file_location(name, str(so))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    os.environ.setdefault("MAX_JOBS", "4")
    names = build(a.reference, a.verbose)
    print("built:", names)
    sys.exit(0 if names else 1)
