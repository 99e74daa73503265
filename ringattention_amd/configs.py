"""The five synthetic workloads the engine is specified on (shape, dtype, seed, sigma)."""
from dataclasses import dataclass


@dataclass(frozen=True)
class Workload:
    name: str
    batch: int
    heads: int
    dim: int
    npes: int       # P virtual ring ranks
    chunk: int      # tokens per rank
    dtype: str      # "fp16" | "bf16"
    seed: int
    causal: bool
    sigma_qk: float = 1.0
    sigma_v: float = 1.0
    graph: bool = False

    @property
    def seq(self):
        return self.npes * self.chunk

    @property
    def rows(self):
        return self.batch * self.heads * self.seq

    @property
    def flops(self):
        """Algorithmic FLOP: 4 * B * H * d * (visible (q, k) pairs)."""
        s = self.seq
        pairs = s * (s + 1) // 2 if self.causal else s * s
        return 4 * self.batch * self.heads * self.dim * pairs


WORKLOADS = {
    "cfg1": Workload("cfg1", 1, 1, 64, 4, 128, "fp16", 0, False),
    "cfg2": Workload("cfg2", 1, 8, 64, 8, 1024, "fp16", 1, False),
    "cfg3": Workload("cfg3", 4, 16, 128, 32, 512, "fp16", 2, False, graph=True),
    "cfg4": Workload("cfg4", 1, 32, 128, 8, 4096, "bf16", 3, True),
    "cfg5": Workload("cfg5", 1, 16, 128, 16, 8192, "fp16", 4, False, sigma_qk=3.0),
}
