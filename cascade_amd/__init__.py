"""cascade_amd: MI355X (gfx950) per-partition suffix sort by prefix doubling, behind a C ABI.

The compute lives in libcascade_hip.so (hand-written HIP, include/cascade_hip.h); this package is the thin
host-side mirror of the reference's builder interface for that one path.
"""
from . import _native, workloads
from .gpu_saca import GPU_SACA, PartitionSorter, output_cut, pack_keys, partition_ids, sort_partition, sort_partitions, stage_slab

__all__ = ["GPU_SACA", "PartitionSorter", "output_cut", "pack_keys", "partition_ids", "sort_partition", "sort_partitions", "stage_slab", "workloads", "_native"]
