"""An independent restatement of the reference's per-token decode step, used to
pin the CPU checker's two decode loops (`ko_gemma_forward`, `ko_gemma4_forward`).

It follows the reference's OTHER formulation of the step, the branch for mixed
weight packings in crates/ksearch_gemma/src/gemma_prim.rs: one `rmsnorm`, then
three separate q / k / v GEMVs (:566-579); `rmsnorm_add` after the attention
output projection, a separate `rmsnorm` in front of gate and up, `gelu_mul`,
down, `rmsnorm_add` (:1100-1150); the per-layer-embedding prepass (:845-878)
and tail (:1166-1200); the window and cache-source rules (:1010-1017 and
crates/ksearch_gemma/src/lib.rs:137-162).  All arithmetic is float64 numpy on
dequantized weight matrices, softmax attention is the textbook form over the
dequantized cache; only the byte-level pieces that single-op tests already pin
are taken from the checker (block dequantization, the Q4_0 packer).

Q4_0 re-quantization of K and V is the one place where f64 and sequential-f32
arithmetic may legitimately part ways (a value on a code boundary), so the
restatement packs its own rows, reports how they differ from the rows handed
in, and then attends over the rows handed in.
"""
from __future__ import annotations

import numpy as np

import oracle

Q4K, Q5K, Q6K, Q40 = oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q40


def deq_matrix(dtype, w, rows, cols) -> np.ndarray:
    return oracle.dequant(dtype, w, rows * cols).astype(np.float64).reshape(rows, cols)


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x) + eps)


def rope_table(max_seq, hd, theta, rope_angles):
    """gemma_prim.rs:33-56: freq in f64 then cast to f32, angle = pos*freq in f32; cos || sin halves;
    pairs past `rope_angles` are the identity."""
    half = hd // 2
    t = np.zeros((max_seq, hd), dtype=np.float64)
    t[:, :half] = 1.0
    for i in range(min(rope_angles, half)):
        freq = np.float32(1.0 / (float(theta) ** ((2 * i) / hd)))
        ang = (np.arange(max_seq, dtype=np.float32) * freq).astype(np.float32)
        t[:, i] = np.cos(ang.astype(np.float64))
        t[:, half + i] = np.sin(ang.astype(np.float64))
    return t


def rope(x, row):
    """lower.rs:4356-4435: out[k] = u cos - v sin, out[half+k] = u sin + v cos with u = x[k], v = x[half+k]."""
    half = x.size // 2
    u, v, c, s = x[:half], x[half:], row[:half], row[half:]
    return np.concatenate([u * c - v * s, u * s + v * c])


def gelu_mul(g, u):
    """lower.rs:2926-2955."""
    ax = np.clip(g, -20.0, 20.0)
    return 0.5 * ax * (1.0 + np.tanh(0.79788456 * (ax + 0.044715 * ax ** 3))) * u


class Restatement:
    """cfg / weights as for `oracle.Gemma4` (the plain loop is the special case built by `from_plain`)."""

    def __init__(self, cfg: dict, weights: dict):
        self.c, self.pos = dict(cfg), 0
        c, g = self.c, weights["globals"]
        h, n = c["hidden"], c["n_layers"]
        self.embd = deq_matrix(g["dt_embd"], g["token_embd"], c["vocab"], h)
        self.output_norm = g["output_norm"].astype(np.float64)
        self.pd = c["ple_dim"]
        if self.pd:
            pt = n * self.pd
            self.ple_embd = deq_matrix(g["dt_ple"], g["ple_embd"], c["vocab"], pt)
            self.ple_proj = deq_matrix(g["dt_ple_proj"], g["ple_model_proj"], pt, h)
            self.ple_norm = g["ple_proj_norm"].astype(np.float64)
        self.L = []
        owners = max(n - c["shared_kv_layers"], 0)
        for i, lw in enumerate(weights["layers"]):
            swa = bool(lw["is_swa"])
            hd = c["hd_swa"] if swa else c["hd_full"]
            qd, kvd, f = c["n_q"] * hd, c["n_kv"] * hd, lw["ffn"]
            d = dict(swa=swa, hd=hd, owns=i < owners, scale=float(lw.get("layer_scale", 1.0)),
                     wq=deq_matrix(lw["dt_q"], lw["wq"], qd, h), wo=deq_matrix(lw["dt_o"], lw["wo"], h, qd),
                     wgate=deq_matrix(lw["dt_gate"], lw["wgate"], f, h), wup=deq_matrix(lw["dt_up"], lw["wup"], f, h),
                     wdown=deq_matrix(lw["dt_down"], lw["wdown"], h, f))
            if d["owns"]:
                d["wk"] = deq_matrix(lw["dt_k"], lw["wk"], kvd, h)
                d["wv"] = deq_matrix(lw["dt_v"], lw["wv"], kvd, h)
            if self.pd:
                d["inp_gate"] = deq_matrix(lw["dt_inp_gate"], lw["inp_gate"], self.pd, h)
                d["proj"] = deq_matrix(lw["dt_proj"], lw["proj"], h, self.pd)
            for name in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm", "post_norm"):
                if lw.get(name) is not None:
                    d[name] = lw[name].astype(np.float64)
            self.L.append(d)
        for i, d in enumerate(self.L):      # crates/ksearch_gemma/src/lib.rs:151-162
            d["src"] = i if d["owns"] else next(
                (j for j in range(i - 1, -1, -1) if self.L[j]["owns"] and self.L[j]["swa"] == d["swa"]), 0)
        self.rope_swa = rope_table(c["max_seq"], c["hd_swa"], c["rope_theta_swa"], c["hd_swa"] // 2)
        self.rope_full = rope_table(c["max_seq"], c["hd_full"], c["rope_theta_full"],
                                    int(np.float32(c["hd_full"]) * np.float32(c["partial_rotary"])) // 2)
        # the cache: dequantized rows, [layer][which][pos] -> f64[n_kv*hd]
        self.cache = [[{}, {}] for _ in self.L]

    @classmethod
    def from_plain(cls, cfg: dict, w: dict):
        """The synthetic shape's loop: every layer owns a full-attention cache, nothing else."""
        c4 = dict(n_layers=cfg["n_layers"], hidden=cfg["hidden"], n_q=cfg["n_q"], n_kv=cfg["n_kv"], vocab=cfg["vocab"],
                  max_seq=cfg["max_seq"], hd_swa=cfg["hd"], hd_full=cfg["hd"], sliding_window=1 << 30, shared_kv_layers=0,
                  ple_dim=0, eps=cfg["eps"], softcap=cfg["softcap"], rope_theta_swa=cfg["rope_theta"],
                  rope_theta_full=cfg["rope_theta"], partial_rotary=1.0, attn_scale=cfg["attn_scale"])
        layers = [dict(lw, is_swa=0, ffn=cfg["ffn"], layer_scale=1.0,
                       **{k: Q4K for k in ("dt_q", "dt_k", "dt_v", "dt_o", "dt_gate", "dt_up", "dt_down")})
                  for lw in w["layers"]]
        return cls(c4, dict(layers=layers, globals=dict(token_embd=w["token_embd"], dt_embd=Q6K,
                                                        output_norm=w["output_norm"])))

    def forward(self, token: int, rows):
        """One token.  `rows[layer][which]` are the packed Q4_0 rows to attend over for this position (None for
        layers that append nothing).  Returns (logits, hidden, own_rows) where own_rows has the same layout and
        holds what this restatement packed itself."""
        c, eps, pos = self.c, self.c["eps"], self.pos
        h = c["hidden"]
        x = np.sqrt(np.float32(h)).astype(np.float64) * self.embd[token]
        if self.pd:
            tok = np.sqrt(np.float32(self.pd)).astype(np.float64) * self.ple_embd[token]
            tmp = (self.ple_proj @ x).reshape(c["n_layers"], self.pd)
            ctx = np.stack([rms(r, eps) * self.ple_norm for r in tmp]).reshape(-1)
            ple_ctx = float(np.float32(np.sqrt(0.5))) * (ctx + tok)
        own_rows = []
        for l, d in enumerate(self.L):
            hd, n_q, n_kv = d["hd"], c["n_q"], c["n_kv"]
            rrow = (self.rope_swa if d["swa"] else self.rope_full)[pos]
            x2 = rms(x, eps) * d["attn_norm"]
            q = (d["wq"] @ x2).reshape(n_q, hd)
            q = np.stack([rope(rms(qh, eps) * d["q_norm"], rrow) for qh in q])
            if d["owns"]:
                k = (d["wk"] @ x2).reshape(n_kv, hd)
                v = (d["wv"] @ x2).reshape(n_kv, hd)
                k = np.concatenate([rope(rms(kh, eps) * d["k_norm"], rrow) for kh in k])
                v = np.concatenate([rms(vh, eps) for vh in v])          # no weight on V
                mine = [oracle.pack_q40(k.astype(np.float32)), oracle.pack_q40(v.astype(np.float32))]
                own_rows.append(mine)
                use = mine if rows[l] is None else rows[l]      # no rows handed in: attend over the own ones
                for which in (0, 1):
                    self.cache[l][which][pos] = oracle.dequant(Q40, use[which], n_kv * hd).astype(np.float64)
            else:
                own_rows.append(None)
            kv_len = pos + 1
            start = max(kv_len - c["sliding_window"], 0) if d["swa"] else 0
            K = np.stack([self.cache[d["src"]][0][t] for t in range(start, kv_len)]).reshape(-1, n_kv, hd)
            V = np.stack([self.cache[d["src"]][1][t] for t in range(start, kv_len)]).reshape(-1, n_kv, hd)
            att = np.empty((n_q, hd))
            for hq in range(n_q):
                kvh = hq // (n_q // n_kv)
                s = (K[:, kvh, :] @ q[hq]) * float(np.float32(c["attn_scale"]))
                p = np.exp(s - s.max())
                att[hq] = (p @ V[:, kvh, :]) / p.sum()
            x2 = d["wo"] @ att.reshape(-1)
            x = x + rms(x2, eps) * d["post_attn_norm"]
            x2 = rms(x, eps) * d["ffn_norm"]
            ff = gelu_mul(d["wgate"] @ x2, d["wup"] @ x2)
            x2 = d["wdown"] @ ff
            x = x + rms(x2, eps) * d["post_ffw_norm"]
            if self.pd:
                u = gelu_mul(d["inp_gate"] @ x, ple_ctx[l * self.pd:(l + 1) * self.pd])
                x2 = d["proj"] @ u
                x = float(np.float32(d["scale"])) * (x + rms(x2, eps) * d["post_norm"])
        self.pos += 1
        logits = self.embd @ (rms(x, eps) * self.output_norm)
        return logits, x, own_rows
