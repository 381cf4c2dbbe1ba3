"""PyTorch counterpart of the reference's Keras optimizer (keras/comprex_optimizer.py:7-170):
momentum SGD whose gradient exchange is one of the compressed allreduce schedules.

Per step and rank (blob mode, keras/comprex_optimizer.py:97-133): every gradient is clipped to
`pre_clipnorm`, turned into a local momentum term `m = momentum * m + lr * g`, all terms are
concatenated into ONE flat device buffer, the allreduce works in place on that buffer (device
pointer handed straight to the C ABI), the result is divided by the number of ranks, and
`w = (1 - weight_decay) * w - avg_m`.  With a single rank nothing is exchanged and, as in the
reference (:134-141,155-163), the update is `m = momentum * m + g; w = (1 - wd) * w - m`.
"""
import torch

from . import pygpi

_SCHEDULES = {
    "comprex_alltoone": pygpi.Comprex_AllToOneAllreduce,
    "comprex_ring": pygpi.Comprex_RingAllreduce,
    "comprex_bigring": pygpi.Comprex_BigRingAllreduce,
}


class ComprexOptimizer(torch.optim.Optimizer):
    def __init__(self, params, gaspi_env, learning_rate=0.01, momentum=0.9, compression_ratio=0.01,
                 allreduce_type="comprex_bigring", size_factor=1.0, pre_clipnorm=5.0, weight_decay=0.0):
        if not 0 <= momentum <= 1:
            raise ValueError("`momentum` must be between [0, 1].")
        if allreduce_type not in _SCHEDULES:
            raise ValueError("AllreduceOp with name %s is not known!" % allreduce_type)
        super().__init__(params, dict(lr=learning_rate, momentum=momentum, weight_decay=weight_decay))
        self.gaspi_env = gaspi_env
        self.compression_ratio = compression_ratio
        self.size_factor = size_factor
        self.allreduce_type = allreduce_type
        self.pre_clipnorm = pre_clipnorm
        self.allreduce = None
        self.blob = None

    def set_compression_ratio(self, compression_ratio):
        self.compression_ratio = compression_ratio
        if self.allreduce is not None:
            self.allreduce.set_compression_ratio(compression_ratio)

    def _create_allreduce(self, size):
        ar = _SCHEDULES[self.allreduce_type](self.gaspi_env)
        if self.allreduce_type == "comprex_alltoone":
            ar.setup_connections(size, 1, 0, self.compression_ratio, self.size_factor)
        else:
            ar.setup_connections(size, 1, self.compression_ratio, self.size_factor)
        return ar

    @torch.no_grad()
    def step(self):
        ranks = self.gaspi_env.get_ranks()
        entries = []
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                state = self.state[p]
                if "momentum" not in state:
                    state["momentum"] = torch.zeros_like(p)
                entries.append((p, group, state["momentum"]))
        if ranks == 1:
            for p, group, mom in entries:
                mom.mul_(group["momentum"]).add_(p.grad)
                p.mul_(1 - group["weight_decay"]).sub_(mom)
            return
        total = sum(p.numel() for p, _, _ in entries)
        if self.blob is None or self.blob.numel() != total:
            self.blob = torch.empty(total, dtype=torch.float32, device=entries[0][0].device)
            self.allreduce = self._create_allreduce(total)
        off = 0
        for p, group, mom in entries:
            g = p.grad
            norm = g.norm()
            if norm > self.pre_clipnorm:  # tf.clip_by_norm
                g = g * (self.pre_clipnorm / norm)
            mom.mul_(group["momentum"]).add_(g, alpha=group["lr"])
            self.blob[off:off + p.numel()].copy_(mom.reshape(-1))
            off += p.numel()
        self.allreduce.apply(self.blob)  # in place, on the device
        self.blob.div_(ranks)
        off = 0
        for p, group, _ in entries:
            p.mul_(1 - group["weight_decay"]).sub_(self.blob[off:off + p.numel()].view_as(p))
            off += p.numel()
