"""Seeded synthetic inputs of the benchmark configurations (numpy, PCG64).

One generator per tensor kind; every config uses `rng(cfg, salt)` =
numpy.random.default_rng([0xA11A, cfg, salt]) so tests, smoke and the benchmark
draw identical bytes.  Shapes and distributions:
  * activations ~ N(0,1) (f32, or rounded once to fp16), gamma ~ N(1, 0.05) f32;
  * Q8_0 table: per 34-byte block an f16 scale |N(0,0.02)|/127 (about a third are
    f16 subnormals) and 32 int8 quants uniform in [-127,127];
  * Q4_K table: per 144-byte super-block d, dmin = f16(|N(0,0.02)|/63), 12 uniform
    random scale bytes (=> random 6-bit scales and mins), 128 uniform nibble bytes;
  * router logits ~ N(0,1) f32.
"""
import numpy as np

MODELS = {
    "qwen3-0.6b": dict(hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, vocab=151936, eps=1e-6, theta=1e6),
    "qwen3-32b": dict(hidden=5120, n_q=64, n_kv=8, head_dim=128, ffn=25600, vocab=151936, eps=1e-6, theta=1e6),
    "qwen3-30b-a3b": dict(hidden=2048, n_expert=128, top_k=8, moe_ffn=768, eps=1e-6),
}


def rng(cfg, salt=0):
    return np.random.default_rng([0xA11A, int(cfg), int(salt)])


def normal_f32(g, shape, mean=0.0, std=1.0):
    return (mean + std * g.standard_normal(shape)).astype(np.float32)


def to_f16_bits(x):
    return x.astype(np.float16).view(np.uint16)


def q8_0_table(g, rows, n_in):
    nb = n_in // 32
    blk = np.empty((rows, nb, 34), np.uint8)
    scale = (np.abs(g.standard_normal((rows, nb))) * 0.02 / 127.0).astype(np.float32).astype(np.float16)
    blk[:, :, 0:2] = scale.view(np.uint8).reshape(rows, nb, 2)
    blk[:, :, 2:] = g.integers(-127, 128, size=(rows, nb, 32), dtype=np.int8).view(np.uint8)
    return blk.reshape(rows, nb * 34)


def q4_k_table(g, rows, n_in):
    nsb = n_in // 256
    blk = g.integers(0, 256, size=(rows, nsb, 144), dtype=np.uint8)
    dd = (np.abs(g.standard_normal((rows, nsb, 2))) * 0.02 / 63.0).astype(np.float32).astype(np.float16)
    blk[:, :, 0:4] = dd.view(np.uint8).reshape(rows, nsb, 4)
    return blk.reshape(rows, nsb * 144)


def layer_inputs(model, rows, salt=0):
    """The inputs of one decoder layer's fused ops at `rows` tokens, f32, from one seeded generator: what both legs of the
    benchmark run on (the device leg narrows the activations to its activation type, the CPU leg takes them as they
    are).  x, delta [rows, hidden]; gamma1, gamma2 [hidden]; q [rows, n_q*hd], k [rows, n_kv*hd]; qw, kw [hd];
    gate, up [rows, ffn]."""
    m = MODELS[model]
    g = rng(2, 1000 + salt)
    H, hd = m["hidden"], m["head_dim"]
    return dict(
        x=normal_f32(g, (rows, H)), delta=normal_f32(g, (rows, H)),
        gamma1=normal_f32(g, H, 1.0, 0.05), gamma2=normal_f32(g, H, 1.0, 0.05),
        q=normal_f32(g, (rows, m["n_q"] * hd)), k=normal_f32(g, (rows, m["n_kv"] * hd)),
        qw=normal_f32(g, hd, 1.0, 0.05), kw=normal_f32(g, hd, 1.0, 0.05),
        gate=normal_f32(g, (rows, m["ffn"])), up=normal_f32(g, (rows, m["ffn"])),
    )
