"""CPU cores for the worker process of each GPU, from the kernel's topology files.

Host-side mirror of tspipe/affinity_manager.py:10-84.  The reference asks
``nvidia-smi topo -m`` for every GPU's "CPU Affinity" column (40-54) and pins
processes with ``taskset`` (73-75); neither exists on a ROCm machine, and TSPipe
calls this before anything else (tspipe/tspipe.py:141-142,
tspipe/gpu_worker.py:600).  Here the same lists come from sysfs: the amdgpu
driver exports one topology node per GPU under
``/sys/class/kfd/kfd/topology/nodes`` (in the order HIP numbers the devices),
each with the PCI address of its device, and that PCI device's
``local_cpulist`` names the cores next to it.  Processes are pinned with
``sched_setaffinity``.  Like the reference's, the map covers every GPU the
machine shows, whatever ``HIP_VISIBLE_DEVICES`` says.

The sharing rule is the reference's (30-37, 56-71): a GPU gets at most four
cores, fewer when other GPUs list the same ones (its list's length divided by
the largest number of GPUs that share one of its cores), taken from the front
of its list, and cores given to one GPU are struck from the lists of the others.
"""
import os
import re
from typing import Dict, List

_KFD_NODES = "class/kfd/kfd/topology/nodes"
_MAX_CORES_PER_GPU = 4


def _node_properties(path: str) -> Dict[str, int]:
    props: Dict[str, int] = {}
    with open(path) as fh:
        for line in fh:
            name, _, value = line.strip().partition(" ")
            if value.strip().lstrip("-").isdigit():
                props[name] = int(value)
    return props


class AffinityManager:
    def __init__(self, process=None):
        """``process``: anything with a ``pid`` (a ``multiprocessing.Process``);
        the calling process when omitted."""
        self.process = process
        self.pid = process.pid if process is not None else os.getpid()

    @staticmethod
    def parse_affinity(affinity: str) -> List[int]:
        """``"0-3,8,10-11"`` -> ``[0, 1, 2, 3, 8, 10, 11]`` (the format of
        ``local_cpulist`` and of nvidia-smi's column alike)."""
        assert re.match(r"^(\d+(-\d+)?)(,\d+(-\d+)?)*$", affinity)
        cores: List[int] = []
        for part in affinity.split(","):
            first, _, last = part.partition("-")
            cores.extend(range(int(first), int(last or first) + 1))
        return cores

    @staticmethod
    def num_cpus_for_gpu(gpu_id: int, affinities: Dict[int, List[int]]) -> int:
        mine = affinities[gpu_id]
        sharers = max(sum(core in cores for cores in affinities.values()) for core in mine)
        return min(len(mine) // sharers, _MAX_CORES_PER_GPU)

    @staticmethod
    def gpu_cpu_lists(sysfs_root: str = "/sys") -> Dict[int, List[int]]:
        """GPU index -> the cores next to that GPU, before any sharing rule."""
        nodes_dir = os.path.join(sysfs_root, _KFD_NODES)
        if not os.path.isdir(nodes_dir):
            raise RuntimeError(f"no amdgpu compute topology under {nodes_dir}: is the amdgpu driver loaded?")
        lists: Dict[int, List[int]] = {}
        for node in sorted((n for n in os.listdir(nodes_dir) if n.isdigit()), key=int):
            props = _node_properties(os.path.join(nodes_dir, node, "properties"))
            if props.get("simd_count", 0) == 0:
                continue  # a CPU node
            location = props.get("location_id", 0)
            address = "%04x:%02x:%02x.%x" % (props.get("domain", 0), (location >> 8) & 0xff, (location >> 3) & 0x1f,
                                             location & 0x7)
            text = ""
            cpulist = os.path.join(sysfs_root, "bus/pci/devices", address, "local_cpulist")
            if os.path.exists(cpulist):
                with open(cpulist) as fh:
                    text = fh.read().strip()
            # a virtual machine may leave the list empty: every core this process may use then
            lists[len(lists)] = AffinityManager.parse_affinity(text) if text else sorted(os.sched_getaffinity(0))
        return lists

    @staticmethod
    def get_gpu_affinity_map(sysfs_root: str = "/sys") -> Dict[int, List[int]]:
        lists = AffinityManager.gpu_cpu_lists(sysfs_root)
        demand = {gpu: AffinityManager.num_cpus_for_gpu(gpu, lists) for gpu in lists}
        left = {gpu: list(cores) for gpu, cores in lists.items()}
        for gpu in sorted(left):
            assert len(left[gpu]) >= demand[gpu]
            chosen = left[gpu][:demand[gpu]]
            for other in left:
                if other != gpu:
                    left[other] = [core for core in left[other] if core not in chosen]
            left[gpu] = chosen
        return left

    def set_affinity(self, cpu_list: List[int]) -> None:
        """Pins the process; like the reference's ``taskset`` call (73-75), a
        refusal (an empty list, cores outside the process's cgroup) is ignored."""
        try:
            os.sched_setaffinity(self.pid, cpu_list)
        except (OSError, ValueError):
            pass

    def set_affinity_for_gpu(self, gpu_id: int, sysfs_root: str = "/sys") -> None:
        self.set_affinity(AffinityManager.get_gpu_affinity_map(sysfs_root)[gpu_id])

    def set_affinity_for_scheduler(self, sysfs_root: str = "/sys") -> None:
        """Everything the GPU workers did not get (tspipe/affinity_manager.py:81-84)."""
        taken = {core for cores in AffinityManager.get_gpu_affinity_map(sysfs_root).values() for core in cores}
        self.set_affinity(sorted(set(range(os.cpu_count())) - taken))

