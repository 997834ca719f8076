"""A second plain Qwen3 pass, independent of ``qwen3_plain`` in source, structure and arithmetic.

``qwen3_plain`` transcribes the reference's CPU backend and runs a sequence whole, with torch in
float32.  This one transcribes the reference's CUDA backend and its model as a list of operations on
named buffers, runs ONE TOKEN AT A TIME against growing lists of keys and values (the way the
reference decodes), in numpy float64, with explicit loops over heads.  Where the two agree, a mistake
in reading the layer order would have had to be made twice in two different shapes; the tests then
mutate this pass (norm after the rotation, another eps, a norm in the wrong place) to show that the
comparison would see such a mistake.

It shares no code with the product or with ``qwen3_plain``.
"""
import json
import math
import os

import numpy as np
from safetensors import safe_open


def _load(folder):
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k).double().numpy()
    return out


def op_embedding(weight, token):
    """src/backends/cuda/native/common.cuh:45-56: output[i] = weight[token * hidden + i]."""
    return weight[token].copy()


def op_rmsnorm(x, weight, eps):
    """src/backends/cuda/native/common.cuh:58-186 over the last axis: scale = rsqrt(sum(x^2) * (1/dims) + eps),
    out = x * scale * w."""
    dims = x.shape[-1]
    scale = 1.0 / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) * (1.0 / dims) + eps)
    return x * scale * weight


def op_linear(x, weight):
    """src/backends/cuda/kernels.cu:62-69 / cublas/sgemm.cu: C[m, n] = sum_k A[m, k] * W[n, k]."""
    return np.einsum("k,nk->n", x, weight)


def op_rope(x, pos, theta):
    """src/backends/cuda/native/common.cu:34-54 with the table of src/utils/constant_table.hpp:28-41:
    rotation_size = head_dim / 2, freq_j = theta^(-j / rotation_size), pairs (j, j + rotation_size)."""
    heads, d = x.shape
    rot = d // 2
    out = np.empty_like(x)
    for j in range(rot):
        freq = np.float32(theta) ** np.float32(-float(j) / float(rot))       # std::pow on floats
        ang = float(np.float32(pos) * np.float32(freq))                      # pos * freq in float32, as the table does
        c, s = math.cos(ang), math.sin(ang)
        v0, v1 = x[:, j], x[:, j + rot]
        out[:, j] = v0 * c - v1 * s
        out[:, j + rot] = v0 * s + v1 * c
    return out


def op_attention(q, keys, values, n_q, n_kv, d):
    """One query token over all keys so far (the newest included: its position is the last).
    src/backends/cuda/native/attention.cu: kv head = head / (num_heads / num_kv_heads) (:121-122), score = dot * scale
    (:156), a key counts when kv_pos <= q_pos (:160), softmax, sum of p * v."""
    per = n_q // n_kv
    scale = 1.0 / math.sqrt(d)
    out = np.zeros((n_q, d))
    for h in range(n_q):
        g = h // per
        scores = np.array([float(np.dot(q[h], k[g])) * scale for k in keys])
        scores -= scores.max()
        p = np.exp(scores)
        p /= p.sum()
        for pc, v in zip(p, values):
            out[h] += pc * v[g]
    return out


def op_swiglu(gate, up):
    """src/backends/cuda/native/common.cu:56-73: (g / (1 + exp(-g))) * u."""
    return (gate / (1.0 + np.exp(-gate))) * up


class SecondQwen3:
    """The operation list of src/models/qwen3.hpp:113-301, buffer by buffer."""

    def __init__(self, folder, qk_norm_after_rope=False, qk_eps=None, post_norm_before_add=False, final_norm=True,
                 embed_scale=1.0):
        with open(os.path.join(folder, "config.json")) as f:
            c = json.load(f)
        self.c = c
        self.w = _load(folder)
        self.n_q, self.n_kv = c["num_attention_heads"], c["num_key_value_heads"]
        self.d = c.get("head_dim", c["hidden_size"] // self.n_q)
        self.eps = c.get("rms_norm_eps", 1e-6)
        self.theta = c.get("rope_theta", 1000000.0)
        if c.get("tie_word_embeddings", False):
            self.w["lm_head.weight"] = self.w["model.embed_tokens.weight"]       # qwen3.hpp:46
        # the mutations that the tests switch on, one at a time
        self.qk_norm_after_rope, self.qk_eps = qk_norm_after_rope, (self.eps if qk_eps is None else qk_eps)
        self.post_norm_before_add, self.final_norm, self.embed_scale = post_norm_before_add, final_norm, embed_scale

    def forward(self, tokens):
        w, c = self.w, self.c
        L = c["num_hidden_layers"]
        k_cache = [[] for _ in range(L)]
        v_cache = [[] for _ in range(L)]
        logits = []
        for pos, tok in enumerate(tokens):
            hidden_states = op_embedding(w["model.embed_tokens.weight"], tok) * self.embed_scale        # :113-119
            for i in range(L):
                b = "model.layers.%d." % i
                norm_1 = op_rmsnorm(hidden_states, w[b + "input_layernorm.weight"], self.eps)            # :127-133
                q = op_linear(norm_1, w[b + "self_attn.q_proj.weight"]).reshape(self.n_q, self.d)        # :138-158
                k = op_linear(norm_1, w[b + "self_attn.k_proj.weight"]).reshape(self.n_kv, self.d)
                v = op_linear(norm_1, w[b + "self_attn.v_proj.weight"]).reshape(self.n_kv, self.d)
                if not self.qk_norm_after_rope:
                    q = op_rmsnorm(q, w[b + "self_attn.q_norm.weight"], self.qk_eps)                      # :161-180
                    k = op_rmsnorm(k, w[b + "self_attn.k_norm.weight"], self.qk_eps)
                q = op_rope(q, pos, self.theta)                                                          # :183-194
                k = op_rope(k, pos, self.theta)
                if self.qk_norm_after_rope:
                    q = op_rmsnorm(q, w[b + "self_attn.q_norm.weight"], self.qk_eps)
                    k = op_rmsnorm(k, w[b + "self_attn.k_norm.weight"], self.qk_eps)
                k_cache[i].append(k)
                v_cache[i].append(v)
                att_output = op_attention(q, k_cache[i], v_cache[i], self.n_q, self.n_kv, self.d)        # :197-205
                att_proj_o = op_linear(att_output.reshape(-1), w[b + "self_attn.o_proj.weight"])         # :207-213
                if self.post_norm_before_add:
                    normed = op_rmsnorm(hidden_states, w[b + "post_attention_layernorm.weight"], self.eps)
                    hidden_states = hidden_states + att_proj_o
                else:
                    hidden_states = hidden_states + att_proj_o                                           # :216-221
                    normed = op_rmsnorm(hidden_states, w[b + "post_attention_layernorm.weight"], self.eps)   # :224-230
                mlp_gate = op_linear(normed, w[b + "mlp.gate_proj.weight"])                              # :233-247
                mlp_up = op_linear(normed, w[b + "mlp.up_proj.weight"])
                swiglu_output = op_swiglu(mlp_gate, mlp_up)                                              # :249-254
                att_proj_o = op_linear(swiglu_output, w[b + "mlp.down_proj.weight"])                     # :257-263
                hidden_states = hidden_states + att_proj_o                                               # :272-277
            if self.final_norm:
                hidden_states = op_rmsnorm(hidden_states, w["model.norm.weight"], self.eps)              # :287-293
            logits.append(op_linear(hidden_states, w["lm_head.weight"]))                                 # :295-301
        return np.stack(logits)
