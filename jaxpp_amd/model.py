"""Layer shapes, parameter initialisation and FLOP accounting for the stage
workloads (host logic, numpy only).

The reference leaves layer arithmetic to the user's model
(examples/basic.py:33-91, README.md:46-72); the three families here are the
ones its examples and the benchmark configurations name.
"""
from __future__ import annotations

import zlib
from dataclasses import asdict, dataclass

import numpy as np


@dataclass(frozen=True)
class LayerSpec:
    family: str                      # "bert" | "decoder" | "llama" | "mixtral"
    hidden: int
    n_heads: int
    ffn: int
    seq: int
    batch: int                       # sequences per microbatch
    n_kv_heads: int | None = None
    head_dim: int | None = None
    causal: bool = False
    rope_theta: float = 5e5
    eps: float = 1e-12
    gelu_tanh: bool = False
    n_experts: int = 0
    top_k: int = 0
    dtype: str = "bf16"              # element type of parameters and activations: "bf16" | "f32"

    @property
    def kvh(self) -> int:
        return self.n_kv_heads or self.n_heads

    @property
    def d(self) -> int:
        return self.head_dim or self.hidden // self.n_heads

    @property
    def tokens(self) -> int:
        return self.seq * self.batch

    @property
    def qkv_width(self) -> int:
        return (self.n_heads + 2 * self.kvh) * self.d

    def as_dict(self) -> dict:
        return asdict(self)

    def param_shapes(self) -> dict:
        h, f = self.hidden, self.ffn
        if self.family in ("bert", "decoder"):
            return {"Wqkv": (h, 3 * h), "bqkv": (3 * h,), "Wo": (h, h), "bo": (h,),
                    "ln1_g": (h,), "ln1_b": (h,), "W1": (h, f), "b1": (f,),
                    "W2": (f, h), "b2": (h,), "ln2_g": (h,), "ln2_b": (h,)}
        if self.family == "llama":
            return {"rms1_g": (h,), "Wqkv": (h, self.qkv_width),
                    "Wo": (self.n_heads * self.d, h), "rms2_g": (h,),
                    "Wgu": (h, 2 * f), "Wd": (f, h)}
        if self.family == "mixtral":
            E = self.n_experts
            return {"rms1_g": (h,), "Wqkv": (h, self.qkv_width),
                    "Wo": (self.n_heads * self.d, h), "rms2_g": (h,),
                    "Wr": (h, E), "Wgu": (E, h, 2 * f), "Wd": (E, f, h)}
        raise ValueError(self.family)

    # -- algorithmic FLOPs: matmuls only, 2*M*N*K; attention halved if causal
    def fwd_flops(self) -> float:
        T, h, f, d = self.tokens, self.hidden, self.ffn, self.d
        qkv = 2.0 * T * h * self.qkv_width
        attn = 4.0 * T * self.seq * self.n_heads * d * (0.5 if self.causal else 1.0)
        out = 2.0 * T * self.n_heads * d * h
        if self.family in ("bert", "decoder"):
            ffn = 4.0 * T * h * f
        elif self.family == "llama":
            ffn = 6.0 * T * h * f
        else:
            ffn = self.top_k * 6.0 * T * h * f + 2.0 * T * h * self.n_experts
        return qkv + attn + out + ffn

    def n_matmul_params(self) -> int:
        return sum(int(np.prod(s)) for k, s in self.param_shapes().items() if len(s) >= 2)


def init_layer_params(spec: LayerSpec, seed: int, layer_index: int,
                      perturb: bool = False) -> dict:
    """Weights ~ N(0, 0.02^2) from PCG64 keyed by (seed, layer, name);
    biases / norm shifts zero and norm gains one, or - with ``perturb`` -
    small random offsets so that tests exercise them.  The router of a
    mixture layer is scaled so its logits are ~N(0, 1) for ~N(0, 1) inputs."""
    out = {}
    for name, shape in spec.param_shapes().items():
        key = zlib.crc32(f"{seed}/{layer_index}/{name}".encode())
        rng = np.random.Generator(np.random.PCG64(key))
        if len(shape) >= 2:
            std = (1.0 / np.sqrt(spec.hidden)) if name == "Wr" else 0.02
            out[name] = (rng.standard_normal(shape, dtype=np.float32) * np.float32(std))
        elif name.endswith("_g"):
            out[name] = np.ones(shape, np.float32)
            if perturb:
                out[name] += 0.1 * rng.standard_normal(shape, dtype=np.float32)
        else:
            out[name] = np.zeros(shape, np.float32)
            if perturb:
                out[name] += 0.02 * rng.standard_normal(shape, dtype=np.float32)
    return out


def boundary_tensor(kind: str, stage: int, mb: int, shape, seed: int = 0) -> np.ndarray:
    """Synthetic stage-boundary tensor ~N(0,1): ``kind`` "x" for an incoming
    activation, "dy" for an incoming cotangent."""
    key = zlib.crc32(f"{seed}/{kind}/{stage}/{mb}".encode())
    rng = np.random.Generator(np.random.PCG64(key))
    return rng.standard_normal(shape, dtype=np.float32)


@dataclass(frozen=True)
class Workload:
    """One benchmark configuration: the layer shape, how many layers each of
    this rank's stages holds, the schedule and which rank is executed."""
    name: str
    layer: LayerSpec
    layers_per_stage: int
    schedule: str
    schedule_kwargs: dict
    n_mubatches: int
    rank: int
    dtype: str = "bf16"

    @property
    def tokens_per_step(self) -> int:
        return self.n_mubatches * self.layer.tokens


def workloads() -> dict:
    bert_s = LayerSpec("bert", 256, 4, 1024, 128, 4)
    bert_l = LayerSpec("bert", 1024, 16, 4096, 512, 8)
    llama8 = LayerSpec("llama", 4096, 32, 14336, 4096, 1, n_kv_heads=8, head_dim=128,
                       causal=True, rope_theta=5e5, eps=1e-5)
    llama70 = LayerSpec("llama", 8192, 64, 28672, 4096, 1, n_kv_heads=8, head_dim=128,
                        causal=True, rope_theta=5e5, eps=1e-5)
    mixtral = LayerSpec("mixtral", 4096, 32, 14336, 4096, 2, n_kv_heads=8, head_dim=128,
                        causal=True, rope_theta=5e5, eps=1e-5, n_experts=8, top_k=2)
    return {
        "cfg1": Workload("cfg1", bert_s, 2, "Std1F1B", {"num_stages": 2}, 8, 0, "f32"),
        "cfg2": Workload("cfg2", bert_l, 6, "Std1F1B", {"num_stages": 4}, 16, 0),
        "cfg3": Workload("cfg3", llama8, 4, "Interleaved1F1B",
                         {"num_stages": 8, "mpmd_dim": 4}, 32, 0),
        "cfg4": Workload("cfg4", llama70, 10, "ZeroBubble", {"num_stages": 8}, 24, 1),
        "cfg5": Workload("cfg5", mixtral, 4, "DualPipeV",
                         {"num_stages": 8, "mpmd_dim": 4}, 16, 0),
    }
