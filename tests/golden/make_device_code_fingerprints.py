"""Writes tests/golden/device_code_<rev>.json: one fingerprint per kernel of the device code that a revision of
this repository compiles to (hipcc -O3 for gfx950, the library's flags).

    python tests/golden/make_device_code_fingerprints.py 62fdaf6

The revision's qwen-kernel_amd/csrc and include directories are taken from the git history into a temporary
directory and compiled there; a kernel's fingerprint is the SHA-1 of its instruction stream with comments,
directives, labels and symbol names removed (tests/test_kernel_resources.py: fingerprints_of).  62fdaf6 is the last
tree whose kernels ran, and passed the GPU tests, on an MI355X: the test that reads the file holds the kernels
the library runs by default to that code, instruction for instruction.  Data only: no source text is kept."""
import concurrent.futures
import glob
import json
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "tests"))
import test_kernel_resources as T  # noqa: E402


def main(rev):
    with tempfile.TemporaryDirectory() as tmp:
        tar = subprocess.run(["git", "-C", ROOT, "archive", rev, "qwen-kernel_amd/csrc", "include"], check=True, capture_output=True).stdout
        subprocess.run(["tar", "-x", "-C", tmp], input=tar, check=True)
        files = sorted(glob.glob(os.path.join(tmp, "qwen-kernel_amd", "csrc", "*.hip")))
        with concurrent.futures.ThreadPoolExecutor(max_workers=7) as pool:
            funcs = {}
            for _, f in pool.map(lambda p: T.compile_file(p, os.path.join(tmp, "include")), files):
                funcs.update(f)
    prints = T.fingerprints_of(funcs)
    out = os.path.join(HERE, f"device_code_{rev}.json")
    with open(out, "w") as f:
        json.dump({"revision": rev, "kernels": dict(sorted(prints.items()))}, f, indent=0)
    print(f"{len(prints)} kernels -> {out}")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "62fdaf6")
