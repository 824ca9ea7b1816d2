"""AffinityManager (tspipe/affinity_manager.py:10-84) over the amdgpu topology files."""
import os
import subprocess
import sys

import pytest

from tspipe_amd.affinity_manager import AffinityManager


def _fake_sysfs(root, gpus):
    """gpus: list of (pci address as (domain, bus, device, function), local_cpulist text).
    Node 0 is a CPU node, as on a real machine."""
    nodes = root / "class/kfd/kfd/topology/nodes"
    (nodes / "0").mkdir(parents=True)
    (nodes / "0" / "properties").write_text("cpu_cores_count 32\nsimd_count 0\nlocation_id 0\ndomain 0\n")
    for i, ((domain, bus, dev, fn), cpulist) in enumerate(gpus, start=1):
        (nodes / str(i)).mkdir()
        (nodes / str(i) / "properties").write_text(
            f"cpu_cores_count 0\nsimd_count 1024\nlocation_id {(bus << 8) | (dev << 3) | fn}\ndomain {domain}\n"
            f"unique_id 6151173044371993893\nname gfx950\n")
        pci = root / "bus/pci/devices" / ("%04x:%02x:%02x.%x" % (domain, bus, dev, fn))
        pci.mkdir(parents=True)
        (pci / "local_cpulist").write_text(cpulist + "\n")
    return str(root)


def test_parse_affinity_lists_and_ranges():
    assert AffinityManager.parse_affinity("0-3,8,10-11") == [0, 1, 2, 3, 8, 10, 11]
    assert AffinityManager.parse_affinity("5") == [5]
    for bad in ("", "a-b", "1-", "1,,2", "0-3 "):
        with pytest.raises(AssertionError):
            AffinityManager.parse_affinity(bad)


def test_map_from_topology_files_and_the_sharing_rule(tmp_path):
    # GPUs 0 and 1 sit at the same 16 cores, GPU 2 at 16 others, GPU 3 (another PCI domain) at 6 of its own
    root = _fake_sysfs(tmp_path, [((0, 0x5d, 0, 0), "0-15"), ((0, 0x6d, 0, 0), "0-15"), ((0, 0x9d, 0, 0), "16-31"),
                                  ((1, 0x05, 0x1f, 7), "40-42,50-52")])
    raw = AffinityManager.gpu_cpu_lists(root)
    assert raw == {0: list(range(16)), 1: list(range(16)), 2: list(range(16, 32)), 3: [40, 41, 42, 50, 51, 52]}
    # two GPUs share every core of GPU 0: 16 // 2 = 8, capped at 4; alone: min(16, 4) and min(6, 4)
    assert [AffinityManager.num_cpus_for_gpu(g, raw) for g in range(4)] == [4, 4, 4, 4]
    # GPU 0 takes the first four, which GPU 1 then no longer has
    assert AffinityManager.get_gpu_affinity_map(root) == {0: [0, 1, 2, 3], 1: [4, 5, 6, 7], 2: [16, 17, 18, 19],
                                                          3: [40, 41, 42, 50]}


def test_few_cores_shared_by_many_gpus(tmp_path):
    # four GPUs on six cores: 6 // 4 = 1 core each
    root = _fake_sysfs(tmp_path, [((0, b, 0, 0), "0-5") for b in (0x10, 0x20, 0x30, 0x40)])
    assert AffinityManager.get_gpu_affinity_map(root) == {0: [0], 1: [1], 2: [2], 3: [3]}
    # partly overlapping lists: the demand follows the most shared core of a GPU's own list
    root2 = _fake_sysfs(tmp_path / "b", [((0, 0x10, 0, 0), "0-7"), ((0, 0x20, 0, 0), "4-11")])
    assert AffinityManager.get_gpu_affinity_map(root2) == {0: [0, 1, 2, 3], 1: [4, 5, 6, 7]}


def test_an_empty_cpu_list_means_every_core_of_the_process(tmp_path):
    root = _fake_sysfs(tmp_path, [((0, 0x5d, 0, 0), "")])
    assert AffinityManager.gpu_cpu_lists(root) == {0: sorted(os.sched_getaffinity(0))}


def test_no_topology_is_an_error_that_names_the_directory(tmp_path):
    with pytest.raises(RuntimeError, match="topology"):
        AffinityManager.get_gpu_affinity_map(str(tmp_path))


_CHILD = """
import os, sys, json
sys.path.insert(0, %r)
from tspipe_amd.affinity_manager import AffinityManager
root = sys.argv[1]
before = sorted(os.sched_getaffinity(0))
m = AffinityManager()
getattr(m, sys.argv[2])(*([0] if sys.argv[2] == "set_affinity_for_gpu" else []), sysfs_root=root)
print(json.dumps({"before": before, "after": sorted(os.sched_getaffinity(0))}))
"""


def _in_child(method, root):
    import json
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _CHILD % repo, root, method], capture_output=True, text=True, check=True)
    return json.loads(out.stdout.strip().splitlines()[-1])


def test_pinning_a_process(tmp_path):
    allowed = sorted(os.sched_getaffinity(0))
    if len(allowed) < 3:
        pytest.skip("needs three cores")
    probe = subprocess.run([sys.executable, "-c", f"import os; os.sched_setaffinity(0, {{{allowed[0]}}})"],
                           capture_output=True)
    if probe.returncode != 0:
        pytest.skip("this sandbox does not let a process change its CPU affinity")
    cpulist = ",".join(str(c) for c in allowed[:2])
    root = _fake_sysfs(tmp_path, [((0, 0x5d, 0, 0), cpulist)])
    got = _in_child("set_affinity_for_gpu", root)
    assert got["after"] == allowed[:2]
    # the scheduler gets what the workers did not (cores the process may not use are refused by the kernel)
    got = _in_child("set_affinity_for_scheduler", root)
    assert got["after"] == [c for c in allowed if c not in allowed[:2]]
    # another process, by its pid
    sleeper = subprocess.Popen([sys.executable, "-c", "import time; time.sleep(30)"])
    try:
        AffinityManager(sleeper).set_affinity(allowed[:1])
        assert sorted(os.sched_getaffinity(sleeper.pid)) == allowed[:1]
        AffinityManager(sleeper).set_affinity([])          # refused by the kernel, ignored like taskset's failure
        assert sorted(os.sched_getaffinity(sleeper.pid)) == allowed[:1]
    finally:
        sleeper.kill()
        sleeper.wait()


@pytest.mark.gpu
def test_map_of_this_machine(device):
    lists = AffinityManager.gpu_cpu_lists()
    assert 0 in lists and lists[0] and all(0 <= c < os.cpu_count() for c in lists[0])
    chosen = AffinityManager.get_gpu_affinity_map()
    assert 1 <= len(chosen[0]) <= 4 and chosen[0] == lists[0][:len(chosen[0])]


def test_pure_functions_against_the_reference_recorded_cases():
    """tests/golden/affinity_cases.json holds what the reference's parse_affinity and
    num_cpus_for_gpu returned or raised (written by tests/golden/make_affinity_fixtures.py)."""
    import json
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "affinity_cases.json")) as fh:
        cases = json.load(fh)

    def attempt(fn, *args):
        try:
            return {"value": fn(*args)}
        except Exception as exc:
            return {"raises": type(exc).__name__}

    assert len(cases["parse"]) >= 14 and len(cases["demand"]) >= 6
    for case in cases["parse"]:
        want = {k: v for k, v in case.items() if k != "text"}
        assert attempt(AffinityManager.parse_affinity, case["text"]) == want, case["text"]
    for case in cases["demand"]:
        lists = {int(g): AffinityManager.parse_affinity(t) for g, t in case["lists"].items()}
        for g, want in case["cores"].items():
            assert attempt(AffinityManager.num_cpus_for_gpu, int(g), lists) == want, (case["lists"], g)
