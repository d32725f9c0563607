"""Tensor lists of the reference's language-model sizes, in optimizer registration order.

Order follows lm_adam_create (lang/lm_adam.c:117-136): the tied head/embedding
matrix, the head bias, then per block the attention matrices, the feed-forward
matrices with their biases and the two LayerNorms.  Tensors are packed with no
padding.  The "baseline" layout is the one the benchmark configurations are
quoted on (fused QKV matrix, QKV and output-projection biases); the "reference"
layout is the reference's own (separate Wq, Wk, Wv, Wo and no attention biases).
Weight decay and twins apply to matrices only in the baseline layout.
"""
from .lib import T_DECAY, T_TWIN

MAT = T_DECAY | T_TWIN
VEC = 0

SIZES = {
    # name: (d_model, heads, d_ff, blocks, vocab)
    "tiny": (64, 4, 256, 2, 256),          # the reference's test model (Makefile:97-114)
    "185m": (1024, 16, 4096, 12, 16384),
    "555m": (1536, 24, 6272, 14, 100000),
    "1p4b": (2048, 32, 8192, 24, 100000),
}


def tensors(size, layout="baseline"):
    """-> list of (name, n, flags)."""
    d, _h, ff, blocks, vocab = SIZES[size]
    out = [("w_head", d * vocab, MAT), ("b_head", vocab, VEC)]
    for b in range(blocks):
        p = "blk%d." % b
        if layout == "baseline":
            out += [(p + "w_qkv", d * 3 * d, MAT), (p + "b_qkv", 3 * d, VEC),
                    (p + "w_o", d * d, MAT), (p + "b_o", d, VEC)]
        else:
            out += [(p + "wq", d * d, MAT), (p + "wk", d * d, MAT),
                    (p + "wv", d * d, MAT), (p + "wo", d * d, MAT)]
        out += [(p + "w1", d * ff, MAT), (p + "b1", ff, VEC),
                (p + "w2", ff * d, MAT), (p + "b2", d, VEC),
                (p + "ln1_g", d, VEC), (p + "ln1_b", d, VEC),
                (p + "ln2_g", d, VEC), (p + "ln2_b", d, VEC)]
    return out


def param_count(size, layout="baseline"):
    return sum(n for _name, n, _f in tensors(size, layout))
