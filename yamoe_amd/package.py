"""Lays the built package out the way the kernel hub expects a drbh/yamoe build (reference tree: build.toml:1-36 and
`build/<variant>/yamoe/`): a directory `build/<variant>/yamoe/` holding the Python modules and the two native
libraries, importable as `yamoe`, plus a `build.toml` that names the ROCm sources.

    python -m yamoe_amd.package [--out DIR]        (default DIR: ./dist)

The variant name follows the hub's pattern torch<MAJOR><MINOR>-cxx11-rocm<MAJOR><MINOR>-x86_64-linux for the torch
that is installed.  Loading the result through the hub's own loader is not exercised here (the loader package is not
part of this image); `import yamoe` from the variant directory is.
"""
import argparse
import os
import re
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
MODULES = ("__init__.py", "_ops.py", "_cabi.py", "layers.py", "workloads.py", "sweep.py", "torch_baseline.py", "reference.py",
           "vendored/__init__.py", "vendored/yamoe_ref.py", "vendored/gpt_oss_mlp.py")
LIBS = ("libyamoe_hip.so", "_yamoe_amd_ops.so")

BUILD_TOML = """[general]
name = "yamoe"
universal = false

[torch]
src = [
  "yamoe_amd/csrc/torch_binding.cpp",
  "include/yamoe_hip.h"
]

[kernel.yamoe]
backend = "rocm"
rocm-archs = ["gfx950"]
depends = ["torch"]
src = [
%s
]
"""


def variant_name():
    import torch
    tv = re.match(r"(\d+)\.(\d+)", torch.__version__)
    hip = getattr(torch.version, "hip", None) or "0.0"
    hv = re.match(r"(\d+)\.(\d+)", hip)
    return "torch%s%s-cxx11-rocm%s%s-x86_64-linux" % (tv.group(1), tv.group(2), hv.group(1), hv.group(2))


def package(out_dir):
    for lib in LIBS:
        if not os.path.exists(os.path.join(HERE, lib)):
            raise FileNotFoundError("%s is missing: run `python -m yamoe_amd.build` first" % lib)
    dst = os.path.join(out_dir, "build", variant_name(), "yamoe")
    os.makedirs(dst, exist_ok=True)
    for name in MODULES + LIBS:
        os.makedirs(os.path.dirname(os.path.join(dst, name)), exist_ok=True)
        shutil.copy2(os.path.join(HERE, name), os.path.join(dst, name))
    csrc = sorted(f for f in os.listdir(os.path.join(HERE, "csrc")) if f.endswith((".hip", ".h")))
    with open(os.path.join(out_dir, "build.toml"), "w") as f:
        f.write(BUILD_TOML % ",\n".join('    "yamoe_amd/csrc/%s"' % c for c in csrc))
    return dst


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="dist")
    a = ap.parse_args(argv)
    print(package(a.out))


if __name__ == "__main__":
    sys.exit(main())
