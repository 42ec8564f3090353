"""Build test-only variants of some sub-graph libraries into tests/launch_shapes/_build/<variant>/.

The shipped libraries pick the kernels of a launch from its size: launches of a few thousand tiles search
their tile boundaries inside the reducer blocks and fold carries and aggregators in one block; larger ones
run the search kernel, one fix-up block per 256 tiles and the final sum.  Inputs small enough for the CPU
oracle only ever take the first route.  The variants built here send small inputs down the other one:

  large   the shipped tile shape, but every launch takes the large-launch route;
  tiny    tiles of 64 threads x 4 items on the large-launch route: a row of a few thousand non-zeros then
          spans more tiles than one fix-up block handles, and a launch has hundreds of tiles.
"""
import os
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

BUILD_DIR = os.path.join(HERE, "_build")
GRAPHS = ["csr_spmv", "spmv_dot", "spring_mass", "swe_rusanov", "system_two_selectors", "op_zoo", "index_spmv",
          "index_sums"]
LARGE_ROUTE = ["-DFLEX_TUNE_INBLOCK_MAX_TILES=0", "-DFLEX_TUNE_SINGLE_FIXUP_MAX_TILES=0"]
VARIANTS = {
    "large": {"policy": None, "flags": LARGE_ROUTE},
    "tiny": {"policy": {"block": 64, "ipt_f32": 4, "ipt_f64": 4}, "flags": LARGE_ROUTE},
}


def library(variant: str, name: str) -> str:
    from flexspmv_amd import graphs
    from flexspmv_amd.build import library_path
    return library_path(graphs.get(name), os.path.join(BUILD_DIR, variant))


def build(force: bool = False):
    from flexspmv_amd import graphs
    from flexspmv_amd.build import compile_graph

    def one(job):
        variant, name = job
        v = VARIANTS[variant]
        return compile_graph(graphs.get(name), out_dir=os.path.join(BUILD_DIR, variant), force=force,
                             policy=v["policy"], extra_flags=v["flags"])

    jobs = [(variant, name) for variant in VARIANTS for name in GRAPHS]
    with ThreadPoolExecutor(max_workers=8) as pool:
        return list(pool.map(one, jobs))


if __name__ == "__main__":
    for lib in build(force="--force" in sys.argv):
        print(lib)
