"""The list of kernel instantiations the tests, the smoke check and the benchmark ask for,
and the ahead-of-time compile of that list.

`kernels.json` (beside this file) holds [generator name, params] pairs.  The build step
compiles each of them with hiprtc for gfx950 into the on-disk code-object cache, so a GPU
run loads code objects instead of compiling.  A kernel that is not listed still works: it
is compiled on first use.

    python -m dlgrad_amd.codegen.manifest --record     re-derive kernels.json by running the
                                                       GPU tests, smoke and benchmark in
                                                       compile-only mode (no GPU needed)
    python -m dlgrad_amd.codegen.manifest --compile    compile everything listed
"""
from __future__ import annotations

import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PATH = os.path.join(HERE, "kernels.json")


def _tuplify(v):
    return tuple(_tuplify(x) for x in v) if isinstance(v, list) else v


def load(path: str = PATH) -> list[tuple[str, tuple]]:
    if not os.path.exists(path):
        return []
    with open(path) as f:
        return [(g, _tuplify(p)) for g, p in json.load(f)]


def merge(entries, path: str = PATH) -> None:
    """Adds (generator, params) pairs to the list at `path` (kernels.json unless told otherwise; sorted, de-duplicated)."""
    cur = {json.dumps([g, p]) for g, p in load(path)}
    cur |= {json.dumps([g, list(p)], default=list) for g, p in entries}
    rows = [json.loads(s) for s in sorted(cur)]            # by their text: parameters of one position may differ in type
    with open(path, "w") as f:
        f.write("[\n" + ",\n".join(json.dumps(r) for r in rows) + "\n]\n")


def _compile_one(job) -> str:
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime import hip
    (gen, params), force = job
    src, name, _ = getattr(K, gen)(*params)
    hip.code_object(src, name, force=force)
    return name


def compile_all(jobs: int = 8, force: bool = False) -> int:
    """Compiles every listed kernel; force=True recompiles the ones already in the cache."""
    entries = load()
    if not entries:
        return 0
    from concurrent.futures import ProcessPoolExecutor
    with ProcessPoolExecutor(max_workers=jobs) as ex:
        names = list(ex.map(_compile_one, [(e, force) for e in entries], chunksize=4))
    return len(names)


def record() -> None:
    env = dict(os.environ, DLGRAD_HIP_COMPILE_ONLY="1", DLGRAD_HIP_MANIFEST=PATH, PYTHONPATH=ROOT)
    cmds = [
        [sys.executable, "-m", "pytest", "tests", "-m", "gpu", "-q", "-p", "no:cacheprovider"],
        [sys.executable, "-c", "import __graft_entry__ as g; g.smoke()"],
        [sys.executable, "bench.py", "--steps", "1", "--warmup", "1", "--no-cpu"],
        [sys.executable, "bench.py", "--steps", "1", "--warmup", "1", "--no-cpu", "--workload", "matmul"],
        [sys.executable, "bench.py", "--steps", "1", "--warmup", "1", "--no-cpu", "--workload", "gpt"],
        [sys.executable, "bench.py", "--steps", "1", "--warmup", "1", "--no-cpu", "--workload", "mlp"],
    ]
    for c in cmds:
        print("+", " ".join(c), flush=True)
        subprocess.run(c, cwd=ROOT, env=env, check=False, stdout=subprocess.DEVNULL)
    print(f"{len(load())} kernels listed in {PATH}")


if __name__ == "__main__":
    if "--record" in sys.argv:
        record()
    if "--compile" in sys.argv or "--record" not in sys.argv:
        print(compile_all(force="--force" in sys.argv), "kernels compiled or found in the cache")
