"""Tensor lists of the workloads: which tensors a model has, in which order and how large.

The order follows the reference's flat pools (include/training/optimizer.h:30-32,
src/model/qwen3.cu:1016-1092): per layer q, k, v, o, gate, up, down, then the embedding,
for the FP16 pool; per layer input_norm, q_norm, k_norm, post_attn_norm, then final_norm,
for the norm weights.  Shapes come from include/model/config.h:6-12 (Qwen3-0.6B defaults).
"""
from collections import namedtuple

DTYPE_F16, DTYPE_F32 = 0, 1
NO_DECAY = 1
FROZEN = 4

# n elements; row_len > 0 marks a 2-D tensor whose rows can be masked (embedding)
TensorSpec = namedtuple("TensorSpec", "name n dtype flags row_len")

QWEN3_0_6B = dict(vocab=151936, hidden=1024, inter=3072, layers=28, q_heads=16, kv_heads=8, head_dim=128,
                  tied=True)
QWEN3_8B = dict(vocab=151936, hidden=4096, inter=12288, layers=36, q_heads=32, kv_heads=8, head_dim=128,
                tied=False)


def qwen3_tensor_list(cfg, norm_dtype=DTYPE_F16, reference_decay_groups=False, freeze_embed=False):
    """All parameter tensors of a Qwen3 model.

    norm_dtype: DTYPE_F16 keeps every tensor FP16 (the benchmark configurations);
    DTYPE_F32 gives the reference's layout, where norm weights and their gradients are FP32.
    reference_decay_groups: embedding and norm tensors get NO_DECAY, as the reference's
    step does (include/training/optimizer.h:131-146); otherwise every tensor decays.
    freeze_embed: the embedding is marked FROZEN (TrainingConfig::freeze_embed,
    include/training/trainer.h:269-277; the SFT main sets it).
    """
    H, I = cfg["hidden"], cfg["inter"]
    q_dim, kv_dim, hd = cfg["q_heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["head_dim"]
    nd = NO_DECAY if reference_decay_groups else 0
    proj, norms = [], []
    for l in range(cfg["layers"]):
        proj += [TensorSpec("layers.%d.q_proj" % l, q_dim * H, DTYPE_F16, 0, H),
                 TensorSpec("layers.%d.k_proj" % l, kv_dim * H, DTYPE_F16, 0, H),
                 TensorSpec("layers.%d.v_proj" % l, kv_dim * H, DTYPE_F16, 0, H),
                 TensorSpec("layers.%d.o_proj" % l, H * q_dim, DTYPE_F16, 0, q_dim),
                 TensorSpec("layers.%d.gate_proj" % l, I * H, DTYPE_F16, 0, H),
                 TensorSpec("layers.%d.up_proj" % l, I * H, DTYPE_F16, 0, H),
                 TensorSpec("layers.%d.down_proj" % l, H * I, DTYPE_F16, 0, I)]
        norms += [TensorSpec("layers.%d.input_norm" % l, H, norm_dtype, nd, 0),
                  TensorSpec("layers.%d.q_norm" % l, hd, norm_dtype, nd, 0),
                  TensorSpec("layers.%d.k_norm" % l, hd, norm_dtype, nd, 0),
                  TensorSpec("layers.%d.post_attn_norm" % l, H, norm_dtype, nd, 0)]
    embed = [TensorSpec("embed_tokens", cfg["vocab"] * H, DTYPE_F16, nd | (FROZEN if freeze_embed else 0), H)]
    if not cfg["tied"]:
        embed.append(TensorSpec("lm_head", cfg["vocab"] * H, DTYPE_F16, 0, H))
    norms.append(TensorSpec("final_norm", H, norm_dtype, nd, 0))
    return proj + embed + norms


def _hash64(seed, idx):
    M = (1 << 64) - 1
    z = (seed + idx * 0x9E3779B97F4A7C15) & M
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & M
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & M
    z ^= z >> 31
    return z


def ragged_tensor_list(count=4096, seed=0x5EED0003):
    """Many small tensors: 60% are 128 or 1024 elements (norm-weight-like, half each), the
    rest log-uniform between 128 and 65,536 elements, sizes not rounded to any multiple."""
    import math
    out = []
    for i in range(count):
        u = _hash64(seed, 2 * i) / 2.0 ** 64
        w = _hash64(seed, 2 * i + 1) / 2.0 ** 64
        if u < 0.3:
            n = 128
        elif u < 0.6:
            n = 1024
        else:
            n = int(round(math.exp(w * math.log(512.0)) * 128.0))
            n = max(128, min(65536, n))
        out.append(TensorSpec("ragged.%d" % i, n, DTYPE_F16, 0, 0))
    return out


def total_elements(specs):
    return sum(s.n for s in specs)
