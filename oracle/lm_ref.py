"""CPU restatement of the reference language model's forward, driven by a state dict.

TEST INFRASTRUCTURE ONLY.  Follows
hierarchical_attention_project/Hierarchical_Transformer_Pretrain.py:331-481 (embedding * sqrt(d)
+ sinusoidal PE, span-node init, per layer: norm_y -> cross_update_Y -> residual, norm1 ->
attention -> residual, norm2 -> FFN -> residual, tied output projection) with the attention
parts taken from oracle/hsa_oracle.py.
"""
import math

import torch
import torch.nn.functional as F

from .hsa_oracle import cross_update_y_ref, span_input_y_ref, update_x_from_y_ref


def lm_forward_ref(sd, tokens, num_heads, num_layers, window_size, activation="relu", dtype=torch.float64):
    sd = {k: v.to(dtype) if v.is_floating_point() else v for k, v in sd.items()}
    d = sd["embedding.weight"].shape[1]
    x = F.embedding(tokens, sd["embedding.weight"]) * math.sqrt(d)
    x = x + sd["pos_encoding.pe"][:, :x.size(1)]
    y = span_input_y_ref(x)
    act = {"relu": F.relu, "gelu": F.gelu}[activation]
    for i in range(num_layers):
        p = "layers.%d." % i
        w = {k[len(p) + len("self_attn."):]: v for k, v in sd.items() if k.startswith(p + "self_attn.")}
        ln = lambda t, n: F.layer_norm(t, (d,), sd[p + n + ".weight"], sd[p + n + ".bias"])
        y = y + cross_update_y_ref(x, ln(y, "norm_y"), w, num_heads)
        nx = ln(x, "norm1")
        x = x + update_x_from_y_ref(nx, y, w, num_heads, window_size, causal=True)
        h = act(F.linear(ln(x, "norm2"), sd[p + "feed_forward.fc1.weight"], sd[p + "feed_forward.fc1.bias"]))
        x = x + F.linear(h, sd[p + "feed_forward.fc2.weight"], sd[p + "feed_forward.fc2.bias"])
    return F.linear(x, sd["embedding.weight"], sd["fc_out.bias"])
