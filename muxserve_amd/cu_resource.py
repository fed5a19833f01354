"""Compute shares of colocated jobs: the scheduler's bookkeeping of the GPU in
ten parts and their translation into compute-unit masks.

The reference divides a GPU's SMs into 10 parts and runs every job in a process
of its own under CUDA MPS with CUDA_MPS_ACTIVE_THREAD_PERCENTAGE = 10 x parts
(muxserve/muxsched/resource.py:15-81 SMPart / SMResource; the launcher sets the
variable at muxserve/muxsched/launcher.py:54-61).  On MI355X a part is a fixed
set of compute units - mask bits [N*p/10, N*(p+1)/10), which the driver spreads
round-robin over the 8 accelerator dies - so a job's share is a real, disjoint
set of compute units rather than a percentage:

  * in one process: a HIP stream restricted to the job's parts
    (ops.CUMaskedStream(parts=...), hipExtStreamCreateWithCUMask);
  * one process per job, as the reference launches them: the HSA_CU_MASK
    environment variable of the child (hsa_cu_mask_env).

CUResource keeps the reference's interface and hand-out order (method names,
which part a request gets, when a part counts as overloaded), so a scheduler
written against SMResource runs against it unchanged.
"""
import random
from typing import Iterable, List

from . import _lib

NUM_PARTS = 10


class CUPart:
    """One tenth of the GPU and the number of jobs that hold it."""

    def __init__(self, id: int):
        self.id = id
        self.ref_count = 0

    def acquire(self):
        self.ref_count += 1

    def release(self):
        self.ref_count -= 1

    def is_idle(self) -> bool:
        return self.ref_count == 0

    def is_overloaded(self) -> bool:
        return self.ref_count > 1

    def __repr__(self):
        return f"CUPart({self.id}, held by {self.ref_count})"


class CUResource:
    """The ten parts: free ones are handed out last-freed first; a request that
    may overload takes, once no part is free, a random part that no more than
    one job holds yet (at most `overload_threshold` such extra parts are
    promised by can_allocate)."""

    def __init__(self, overload_threshold: int = 4):
        self.overload_threshold = overload_threshold
        self._parts = [CUPart(i) for i in range(NUM_PARTS)]
        self.free_sms: List[CUPart] = list(self._parts)
        self.unoverloaded_sms: List[int] = list(range(NUM_PARTS))

    def can_allocate(self, num_sms: int, overload: bool = False) -> bool:
        spare = min(self.overload_threshold, len(self.unoverloaded_sms)) if overload else 0
        return len(self.free_sms) + spare >= num_sms

    def allocate(self, num_sms: int, overload: bool = False) -> List[CUPart]:
        got = []
        for _ in range(num_sms):
            if self.free_sms:
                part = self.free_sms.pop()
            else:
                part = self._parts[random.choice(self.unoverloaded_sms)]
                self.unoverloaded_sms.remove(part.id)
            part.acquire()
            got.append(part)
        return got

    def free(self, sms: Iterable[CUPart]) -> None:
        for part in sms:
            part.release()
            if part.is_idle():
                self.free_sms.append(part)
            if not part.is_overloaded() and part.id not in self.unoverloaded_sms:
                self.unoverloaded_sms.append(part.id)

    @property
    def num_free_sms(self) -> int:
        return len(self.free_sms)

    @property
    def num_overloaded_sms(self) -> int:
        return NUM_PARTS - len(self.unoverloaded_sms)


def part_bits(parts) -> int:
    """Bit p set for every part id p (CUPart objects or ints) of a job's share."""
    bits = 0
    for p in parts:
        i = int(getattr(p, "id", p))
        if not 0 <= i < NUM_PARTS:
            raise ValueError(f"part id {i} outside 0..{NUM_PARTS - 1}")
        bits |= 1 << i
    if bits == 0:
        raise ValueError("a job needs at least one part")
    return bits


def cu_mask_words(parts, num_cus: int) -> List[int]:
    """The compute-unit mask of a share as 32-bit words (word w bit b = compute
    unit 32 w + b), built by the library (mux_cu_parts_mask); no GPU needed."""
    import ctypes
    n_words = (num_cus + 31) // 32
    words = (ctypes.c_uint32 * n_words)()
    rc = _lib.attn().mux_cu_parts_mask(part_bits(parts), int(num_cus), words, n_words)
    if rc <= 0:
        _lib.check_attn(rc if rc < 0 else -1, "mux_cu_parts_mask")
    return [int(w) for w in words]


def enabled_cus(parts, num_cus: int) -> List[int]:
    words = cu_mask_words(parts, num_cus)
    return [i for i in range(num_cus) if (words[i // 32] >> (i % 32)) & 1]


def hsa_cu_mask_env(parts, num_cus: int, gpu_index: int = 0) -> str:
    """Value of HSA_CU_MASK for a child process that is to run on this share of
    GPU `gpu_index` ("<gpu>:<cu ranges>"): what the process-per-job launcher sets
    where the reference sets CUDA_MPS_ACTIVE_THREAD_PERCENTAGE."""
    cus = enabled_cus(parts, num_cus)
    runs, start, prev = [], cus[0], cus[0]
    for c in cus[1:]:
        if c != prev + 1:
            runs.append((start, prev))
            start = c
        prev = c
    runs.append((start, prev))
    return f"{gpu_index}:" + ",".join(str(a) if a == b else f"{a}-{b}" for a, b in runs)
