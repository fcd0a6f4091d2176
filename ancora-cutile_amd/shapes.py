"""Parameter name/shape lists of the model families the optimizer step is sized on.

Names follow the reference's models: `embed, final_norm, layer{i}.{input_ln, post_ln, q_norm,
k_norm, q_proj, k_proj, v_proj, o_proj, gate_proj, up_proj, down_proj}`
(ancora/model/qwen3_model.py:41-46, 15-17) and `layer{i}.ffn.{router, gate_proj, up_proj,
down_proj}` for MoE layers (ancora/model/moe_model.py:51-60). Weights are stored (in, out).
"""


def qwen3_shapes(layers=28, hidden=1024, ffn=3072, q_heads=16, kv_heads=8, head_dim=128,
                 vocab=151936):
    """Qwen3-0.6B-shaped set: 596,049,920 parameters at the defaults (tied embedding)."""
    q, kv = q_heads * head_dim, kv_heads * head_dim
    s = {"embed": (vocab, hidden)}
    for i in range(layers):
        p = f"layer{i}."
        s[p + "input_ln"] = (hidden,)
        s[p + "q_norm"] = (head_dim,)
        s[p + "k_norm"] = (head_dim,)
        s[p + "q_proj"] = (hidden, q)
        s[p + "k_proj"] = (hidden, kv)
        s[p + "v_proj"] = (hidden, kv)
        s[p + "o_proj"] = (q, hidden)
        s[p + "post_ln"] = (hidden,)
        s[p + "gate_proj"] = (hidden, ffn)
        s[p + "up_proj"] = (hidden, ffn)
        s[p + "down_proj"] = (ffn, hidden)
    s["final_norm"] = (hidden,)
    return s


def moe_shapes(layers=16, hidden=1024, dense_ffn=3072, experts=16, expert_ffn=1024, q_heads=16,
               kv_heads=8, head_dim=128, vocab=151936):
    """MoE family: even layers dense, odd layers MoE with stacked [E, K, N] expert tensors and an
    (hidden, E) router."""
    q, kv = q_heads * head_dim, kv_heads * head_dim
    s = {"embed": (vocab, hidden)}
    for i in range(layers):
        p = f"layer{i}."
        s[p + "input_ln"] = (hidden,)
        s[p + "q_norm"] = (head_dim,)
        s[p + "k_norm"] = (head_dim,)
        s[p + "q_proj"] = (hidden, q)
        s[p + "k_proj"] = (hidden, kv)
        s[p + "v_proj"] = (hidden, kv)
        s[p + "o_proj"] = (q, hidden)
        s[p + "post_ln"] = (hidden,)
        if i % 2 == 0:
            s[p + "gate_proj"] = (hidden, dense_ffn)
            s[p + "up_proj"] = (hidden, dense_ffn)
            s[p + "down_proj"] = (dense_ffn, hidden)
        else:
            s[p + "ffn.router"] = (hidden, experts)
            s[p + "ffn.gate_proj"] = (experts, hidden, expert_ffn)
            s[p + "ffn.up_proj"] = (experts, hidden, expert_ffn)
            s[p + "ffn.down_proj"] = (experts, expert_ffn, hidden)
    s["final_norm"] = (hidden,)
    return s
