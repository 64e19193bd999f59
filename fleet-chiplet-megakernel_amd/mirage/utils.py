"""Worker-count heuristic (reference: python/mirage/utils.py:38-101)."""
import torch


def get_configurations_from_gpu(rank: int = 0):
    """Return (num_workers, num_schedulers) for device `rank`.

    The reference reserves 8 CUs for scheduler blocks (240 workers + 8 schedulers on a 256-CU MI350).
    The MI355X megakernel has no scheduler blocks -- scheduling is one thread's work between two
    barriers -- so every CU is a worker and the scheduler count is reported as 0.
    """
    props = torch.cuda.get_device_properties(rank)
    return props.multi_processor_count, 0
