"""Where and how a model runs: device, dtype, and the kernels.

dtype "bfloat16": bf16 weights, activations and cache, fp32 residual stream,
statistics, softmax and logits (the reference's fp16/fp32 split, runtime/src/
lib.rs:4483-4516, with bf16 in fp16's place).  dtype "float32": every tensor
and every operation in fp32, no reduced-precision matrix mode.
"""
import torch

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name):
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype {name} is not supported (bfloat16 or float32)")
        return name
    if name not in _DTYPES:
        raise ValueError(f"dtype '{name}' is not supported (bfloat16 or float32)")
    return _DTYPES[name]


class Runtime:
    """`ops` is the kernel library; by default the HIP one, which refuses to load without a GPU."""

    def __init__(self, dtype="bfloat16", device="cuda:0", ops=None):
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if ops is None:
            from .. import kernels
            ops = kernels.load(self.device)
        self.ops = ops
        self._staging = []
        self._next = 0
        self._widened = {}

    def matrix(self, t):
        """A stored floating-point tensor in the width the kernels compute in (bf16 widens to fp32 exactly)."""
        if t.dtype == self.dtype:
            return t
        key = (t.data_ptr(), tuple(t.shape))
        if key not in self._widened:          # a tied head and its embedding share one converted copy
            self._widened[key] = (t, t.to(self.dtype))
        return self._widened[key][1]

    def download_i32(self, t):
        """Device int32 tensor -> host, asynchronously: returns a function that waits for the copy alone (not for
        work enqueued after it) and gives the values as a list."""
        if self.device.type != "cuda":
            values = t.reshape(-1).tolist()
            return lambda: values
        n = t.numel()
        host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        host.copy_(t.reshape(-1), non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()

        def wait():
            ev.synchronize()
            return host.tolist()
        return wait

    def upload_i32(self, array):
        """Host int32 numpy array -> device tensor (asynchronous from pinned memory on a GPU)."""
        t = torch.from_numpy(array)
        if self.device.type != "cuda":
            return t.clone()
        n = t.numel()
        if not self._staging:
            self._staging = [[torch.empty(4096, dtype=torch.int32, pin_memory=True), None] for _ in range(8)]
        slot = self._staging[self._next]
        self._next = (self._next + 1) % len(self._staging)
        if slot[1] is not None:
            slot[1].synchronize()
        if slot[0].numel() < n:
            slot[0] = torch.empty(max(n, 2 * slot[0].numel()), dtype=torch.int32, pin_memory=True)
        slot[0][:n].copy_(t.reshape(-1))
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        out.copy_(slot[0][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        slot[1] = ev
        return out.reshape(array.shape)
