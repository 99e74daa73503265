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
    half_partials: bool = False   # fp16 per-step partial O (RINGATTN_FLAG_HALF_PARTIALS)

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
    # 1024 short chunk pairs per head: the per-step partials dominate the HBM traffic, so they are
    # kept in the I/O type (fp16: V itself is fp16, no range question), and the loop is graph-replayed
    "cfg3": Workload("cfg3", 4, 16, 128, 32, 512, "fp16", 2, False, graph=True, half_partials=True),
    "cfg4": Workload("cfg4", 1, 32, 128, 8, 4096, "bf16", 3, True),
    "cfg5": Workload("cfg5", 1, 16, 128, 16, 8192, "fp16", 4, False, sigma_qk=3.0),
}
