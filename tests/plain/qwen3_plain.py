"""Plain, slow Qwen3-dense forward pass: whole sequences, no cache, one function per part.

Written from the formulas of the reference engine (spymaster2h/spyinfer); every
function cites the reference file and lines it transcribes.  It shares no code
with the ``spyinfer_amd`` package: weights are read with the ``safetensors``
library, config.json with ``json``.  All arithmetic runs on the CPU in the
dtype of ``compute`` (float32 by default, float64 for tighter comparisons).
"""
import json
import math
import os

import torch
from safetensors.torch import load_file


def linear(x, w):
    """y = x . W^T with W stored [out_features, in_features].

    src/backends/cpu/cpu_operator.cpp:147-156 (dot(input + i*k, weight + j*k, k));
    pinned by test/gt/blas_gemm.hpp:43-47 (sgemm RowMajor, NoTrans, Trans).
    No Qwen3 projection has a bias (src/models/qwen3.hpp:39, 212, 238, 246, 262, 300).
    """
    return x @ w.transpose(0, 1)


def rms_norm(x, w, eps):
    """y_i = (1/sqrt(sum(x^2)/n + eps)) * x_i * w_i over the last dim.

    src/backends/cpu/x64/kernels.cpp:168-180: eps inside the sqrt, the weight
    multiplies as it is (no 1 + w), product order (r*x)*w.
    """
    n = x.shape[-1]
    ss = (x * x).sum(dim=-1, keepdim=True)
    r = 1.0 / torch.sqrt(ss / n + eps)
    return (r * x) * w


def rope_tables(num_pos, head_dim, theta, dtype=torch.float32):
    """cos/sin[p, j] for j < head_dim/2, freq_j = theta^(-j / (head_dim/2)).

    src/utils/constant_table.hpp:28-41.  The reference forms freq and p*freq in
    float32; float64 here is used only when ``dtype`` asks for it.
    """
    half = head_dim // 2
    j = torch.arange(half, dtype=dtype)
    freq = torch.pow(torch.tensor(theta, dtype=dtype), -j / half)
    p = torch.arange(num_pos, dtype=dtype)
    ang = p[:, None] * freq[None, :]
    return torch.cos(ang), torch.sin(ang)


def rope_apply(x, positions, cos, sin):
    """Half-split rotation of every head vector x[..., d].

    src/backends/cpu/cpu_operator.cpp:401-407:
      out[j]        = x[j]*cos[p,j] - x[j+d/2]*sin[p,j]
      out[j + d/2]  = x[j]*sin[p,j] + x[j+d/2]*cos[p,j]
    x: [T, heads, d]; positions: [T] absolute index of each token in its sequence.
    """
    half = x.shape[-1] // 2
    c = cos[positions][:, None, :]
    s = sin[positions][:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1)


def attention(q, k, v, window=None):
    """Causal grouped-query attention of one whole sequence, no cache.

    src/backends/cpu/cpu_attention.cpp:59 (scale = 1/sqrt(d), applied after the
    dot product :110), :96 (kv head = h * n_kv / n_q), :98-104 (key c is masked
    when c > position of the query), :113-124 (softmax), :126-135 (sum p_c * v_c).
    q: [T, n_q, d]; k, v: [T, n_kv, d].  ``window`` (not a reference feature; it
    is here to pin the window option of the attention part) keeps only the keys
    c with p - window < c <= p.
    """
    T, n_q, d = q.shape
    n_kv = k.shape[1]
    scale = 1.0 / math.sqrt(d)
    out = torch.zeros_like(q)
    pos = torch.arange(T)
    masked = pos[None, :] > pos[:, None]
    if window is not None:
        masked = masked | (pos[None, :] <= pos[:, None] - window)
    for h in range(n_q):
        g = h * n_kv // n_q
        scores = (q[:, h, :] @ k[:, g, :].transpose(0, 1)) * scale
        scores = scores.masked_fill(masked, float("-inf"))
        m = scores.max(dim=-1, keepdim=True).values
        e = torch.exp(scores - m)
        p = e / e.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def swiglu(gate, up):
    """(g / (1 + exp(-g))) * u.  src/backends/cpu/x64/kernels.cpp:242-247."""
    return (gate / (1.0 + torch.exp(-gate))) * up


def embedding(ids, table):
    """h[t, :] = E[id[t], :], no scaling.  src/backends/cpu/cpu_operator.cpp:251-266."""
    return table[ids]


class PlainQwen3:
    """Reads a model folder and runs whole sequences.  Layer order:
    src/models/qwen3.hpp:122-278 (block) and :283-301 (final norm + lm_head)."""

    def __init__(self, folder, compute=torch.float32, config=None, weights=None):
        """``folder``: a model folder; or None with ``config`` (the config.json keys) and ``weights`` (name -> tensor)
        given directly, for models that are never written to disk."""
        if folder is not None:
            with open(os.path.join(folder, "config.json")) as f:
                c = json.load(f)
        else:
            c = dict(config)
        self.c = c
        self.compute = compute
        self.n_q = c["num_attention_heads"]
        self.n_kv = c["num_key_value_heads"]
        # src/models/model_config.hpp:42: head_dim falls back to hidden/n_q
        self.d = c.get("head_dim", c["hidden_size"] // self.n_q)
        self.eps = c.get("rms_norm_eps", 1e-6)
        self.theta = c.get("rope_theta", 1000000.0)
        self.L = c["num_hidden_layers"]
        if weights is None:
            weights = load_file(os.path.join(folder, "model.safetensors"))
        self.w = {k: v.to("cpu", compute) for k, v in weights.items()}
        # src/models/qwen3.hpp:46: a tied model uses the embedding as lm_head
        if c.get("tie_word_embeddings", False):
            self.w["lm_head.weight"] = self.w["model.embed_tokens.weight"]
        self._tables = None

    def tables(self, n):
        if self._tables is None or self._tables[0].shape[0] < n:
            cos, sin = rope_tables(max(n, 1), self.d, self.theta, torch.float32 if self.compute == torch.float32 else self.compute)
            self._tables = (cos.to(self.compute), sin.to(self.compute))
        return self._tables

    def block(self, h, i, positions, cos, sin, window=None):
        w = self.w
        p = "model.layers.%d." % i
        T = h.shape[0]
        n1 = rms_norm(h, w[p + "input_layernorm.weight"], self.eps)                # qwen3.hpp:127-133
        q = linear(n1, w[p + "self_attn.q_proj.weight"]).view(T, self.n_q, self.d)   # :138-158
        k = linear(n1, w[p + "self_attn.k_proj.weight"]).view(T, self.n_kv, self.d)
        v = linear(n1, w[p + "self_attn.v_proj.weight"]).view(T, self.n_kv, self.d)
        q = rms_norm(q, w[p + "self_attn.q_norm.weight"], self.eps)                # :161-180, before RoPE
        k = rms_norm(k, w[p + "self_attn.k_norm.weight"], self.eps)
        q = rope_apply(q, positions, cos, sin)                                     # :183-194
        k = rope_apply(k, positions, cos, sin)
        a = attention(q, k, v, window).reshape(T, self.n_q * self.d)               # :197-205
        h = h + linear(a, w[p + "self_attn.o_proj.weight"])                        # :207-221
        n2 = rms_norm(h, w[p + "post_attention_layernorm.weight"], self.eps)       # :224-230
        g = linear(n2, w[p + "mlp.gate_proj.weight"])                              # :233-247
        u = linear(n2, w[p + "mlp.up_proj.weight"])
        f = linear(swiglu(g, u), w[p + "mlp.down_proj.weight"])                    # :249-263
        return h + f                                                               # :272-277

    def forward(self, tokens, first_position=0):
        """Logits [T, vocab] at every position of one sequence given whole.

        ``first_position`` shifts all positions (only distances may matter)."""
        ids = torch.as_tensor(tokens, dtype=torch.long)
        T = ids.shape[0]
        positions = torch.arange(T) + first_position
        cos, sin = self.tables(T + first_position)
        h = embedding(ids, self.w["model.embed_tokens.weight"])                    # :114-119
        for i in range(self.L):
            h = self.block(h, i, positions, cos, sin)
        n3 = rms_norm(h, self.w["model.norm.weight"], self.eps)                    # :287-293
        return linear(n3, self.w["lm_head.weight"])                                # :295-301

    def greedy(self, tokens, n_new):
        """Greedy continuation; first maximum wins (src/engine/model_runner.cpp:131)."""
        toks = list(tokens)
        out = []
        for _ in range(n_new):
            nxt = int(torch.argmax(self.forward(toks)[-1]))
            out.append(nxt)
            toks.append(nxt)
        return out
