"""The kernel libraries' build folder (no GPU, nothing is compiled here)."""
from concurrent.futures import ThreadPoolExecutor

from jax_vllm_amd.ops import library


def test_parallel_builds_agree_on_one_folder():
    """``build_all`` compiles the head sizes in parallel threads and each asks where the libraries live:
    every answer is the same folder (a probe file that one thread removed under another once sent
    some of them to the temporary folder, and their libraries were built again at every call)."""
    library._build_dir = None
    with ThreadPoolExecutor(16) as ex:
        found = set(ex.map(lambda _: library.build_dir(), range(64)))
    assert len(found) == 1
    assert not list(found.pop().glob(".w*"))          # no probe file left behind
