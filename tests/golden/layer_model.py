"""Small synthetic models with quantised weights, rebuilt bit for bit from a seed.

Shared by make_layer_fixture.py (which runs them through the unmodified reference CPU backend and
stores the logits) and by the tests (which run the same models through the oracle and the GPU
library).  Only integer arithmetic and single IEEE operations are used, so the bytes do not depend
on the numpy version.

A tensor is (type, uint8 array of its bytes, n_in, n_out) with the reference's type numbers
(reference: src/common.h:47-54) and block layouts (reference: src/quant.h:14-43).
"""
import numpy as np

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K = 0, 1, 8, 12, 13, 14
BLOCK = {F32: (1, 4), F16: (1, 2), Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}
TYPE_NAME = {F32: "F32", F16: "F16", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K"}


class Stream:
    """splitmix64 counter stream."""

    def __init__(self, seed):
        self.ctr = np.uint64(seed)

    def u64(self, n):
        with np.errstate(over="ignore"):
            z = self.ctr + (np.arange(1, n + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
            self.ctr = z[-1] if n else self.ctr
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            return z ^ (z >> np.uint64(31))

    def bytes(self, n):
        return self.u64((n + 7) // 8).view(np.uint8)[:n].copy()

    def unit(self, n):
        """n doubles in [0, 1), multiples of 2^-24."""
        return (self.u64(n) >> np.uint64(40)).astype(np.float64) / 16777216.0

    def sym(self, n, amp):
        """n fp32 values in [-amp, amp)."""
        return ((self.unit(n) * 2.0 - 1.0) * amp).astype(np.float32)


def _half_bytes(x):
    return np.asarray(x, np.float64).astype(np.float16).view(np.uint8).reshape(-1, 2)


def make_tensor(rs, wtype, n_in, n_out, std=0.04):
    """Random rows of the given type whose decoded values have roughly the given spread.
    Every byte that is not a block's fp16 scale is random, so every packing path is exercised
    (six-bit pairs of both kinds, fifth bits, signed scales, subnormal scales)."""
    per, nbytes = BLOCK[wtype]
    assert n_in % per == 0
    nb = n_in // per * n_out
    if wtype == F32:
        return (wtype, rs.sym(n_in * n_out, std * 1.7).view(np.uint8).copy(), n_in, n_out)
    if wtype == F16:
        return (wtype, rs.sym(n_in * n_out, std * 1.7).astype(np.float16).view(np.uint8).copy(), n_in, n_out)
    raw = rs.bytes(nb * nbytes).reshape(nb, nbytes)
    u = rs.unit(nb)
    if wtype == Q8_0:
        raw[:, 0:2] = _half_bytes(std / 74.0 * (0.5 + u))
    elif wtype == Q4_K:
        d = std / 166.0 * (0.5 + u)
        raw[:, 0:2] = _half_bytes(d)
        raw[:, 2:4] = _half_bytes(d * 7.5 * (0.8 + 0.4 * rs.unit(nb)))
    elif wtype == Q5_K:
        d = std / 340.0 * (0.5 + u)
        raw[:, 0:2] = _half_bytes(d)
        raw[:, 2:4] = _half_bytes(d * 15.5 * (0.8 + 0.4 * rs.unit(nb)))
    elif wtype == Q6_K:
        raw[:, 208:210] = _half_bytes(std / 1369.0 * (0.5 + u))   # (mostly fp16 subnormals)
    return (wtype, raw.reshape(-1).copy(), n_in, n_out)


VARIANTS = {
    # arch decides the rotary pairing (reference: src/model_common.cpp:30-34)
    "qwen2": dict(arch="qwen2", seed=101, n_embd=512, n_head=4, n_kv=2, head_dim=128, n_ff=768, n_layer=2,
                  n_vocab=96, n_rot=128, theta=1.0e6, eps=1.0e-6, bias=True, qk_norm=False, factors=False,
                  embd=Q4_K, output=None,
                  types=[dict(wq=Q4_K, wk=Q5_K, wv=Q6_K, wo=Q8_0, ffn_gate=Q4_K, ffn_up=Q5_K, ffn_down=Q6_K),
                         dict(wq=Q6_K, wk=Q8_0, wv=Q4_K, wo=Q5_K, ffn_gate=Q8_0, ffn_up=Q6_K, ffn_down=Q4_K)]),
    "llama": dict(arch="llama", seed=202, n_embd=512, n_head=4, n_kv=4, head_dim=128, n_ff=512, n_layer=2,
                  n_vocab=64, n_rot=64, theta=5.0e5, eps=1.0e-5, bias=False, qk_norm=False, factors=True,
                  embd=F16, output=Q6_K,
                  types=[dict(wq=F16, wk=F32, wv=Q8_0, wo=Q4_K, ffn_gate=Q6_K, ffn_up=Q6_K, ffn_down=Q5_K),
                         dict(wq=Q5_K, wk=Q4_K, wv=F16, wo=F32, ffn_gate=Q4_K, ffn_up=Q4_K, ffn_down=Q8_0)]),
    "qwen3": dict(arch="qwen3", seed=303, n_embd=512, n_head=8, n_kv=2, head_dim=64, n_ff=768, n_layer=2,
                  n_vocab=80, n_rot=64, theta=1.0e6, eps=1.0e-6, bias=False, qk_norm=True, factors=False,
                  embd=Q8_0, output=Q4_K,
                  types=[dict(wq=Q4_K, wk=Q4_K, wv=Q4_K, wo=Q4_K, ffn_gate=Q5_K, ffn_up=Q5_K, ffn_down=Q5_K),
                         dict(wq=Q8_0, wk=Q6_K, wv=Q5_K, wo=Q6_K, ffn_gate=Q6_K, ffn_up=Q8_0, ffn_down=Q6_K)]),
    # NeoX pairing over half the head only (the layout the fused attention call does not take), tied Q6_K embedding,
    # gate and up of one type
    "qwen2p": dict(arch="qwen2", seed=404, n_embd=512, n_head=4, n_kv=1, head_dim=128, n_ff=512, n_layer=2,
                   n_vocab=72, n_rot=64, theta=1.0e4, eps=1.0e-6, bias=True, qk_norm=False, factors=False,
                   embd=Q6_K, output=None,
                   types=[dict(wq=Q5_K, wk=Q5_K, wv=Q5_K, wo=Q6_K, ffn_gate=Q8_0, ffn_up=Q8_0, ffn_down=Q4_K),
                          dict(wq=Q4_K, wk=Q6_K, wv=Q6_K, wo=Q8_0, ffn_gate=Q6_K, ffn_up=Q6_K, ffn_down=Q5_K)]),
    # heads that do not add up to n_embd (n_head * head_dim = 512 < n_embd = 768), with per-head q/k norms: the
    # output projection's rows are shorter than what the reference's decode_layer stages ahead of it
    # (src/model_gpu.cu:284-285)
    "narrow": dict(arch="qwen3", seed=505, n_embd=768, n_head=4, n_kv=2, head_dim=128, n_ff=1024, n_layer=2,
                   n_vocab=88, n_rot=128, theta=1.0e6, eps=1.0e-6, bias=False, qk_norm=True, factors=False,
                   embd=Q4_K, output=Q6_K,
                   types=[dict(wq=Q4_K, wk=Q4_K, wv=Q6_K, wo=Q4_K, ffn_gate=Q4_K, ffn_up=Q4_K, ffn_down=Q6_K),
                          dict(wq=Q8_0, wk=Q5_K, wv=F16, wo=Q6_K, ffn_gate=Q5_K, ffn_up=Q4_K, ffn_down=Q8_0)]),
}
N_TOKENS = 12


def build(name):
    """The model `name` in the form oracle/ref.py's decode_forward takes."""
    c = VARIANTS[name]
    rs = Stream(c["seed"])
    ne, nh, nkv, d, nff = c["n_embd"], c["n_head"], c["n_kv"], c["head_dim"], c["n_ff"]
    hp = dict(arch=c["arch"], n_vocab=c["n_vocab"], n_embd=ne, n_layer=c["n_layer"], n_head=nh, n_kv=nkv,
              head_dim=d, n_ff=nff, n_rot=c["n_rot"], rms_eps=c["eps"], rope_theta=c["theta"],
              neox=1 if c["arch"] in ("qwen2", "qwen3") else 0, freq_factors=None)
    if c["factors"]:
        i = np.arange(c["n_rot"] // 2)
        hp["freq_factors"] = np.clip(1.0 + 7.0 * (i - 10) / 12.0, 1.0, 8.0).astype(np.float32)
    model = dict(hp=hp, layers=[])
    model["token_embd"] = make_tensor(rs, c["embd"], ne, c["n_vocab"], std=1.0)
    model["output"] = make_tensor(rs, c["output"], ne, c["n_vocab"]) if c["output"] is not None else model["token_embd"]
    model["tied_output"] = c["output"] is None
    model["output_norm"] = (1.0 + rs.sym(ne, 0.2)).astype(np.float32)
    for t in c["types"]:
        L = dict(attn_norm=(1.0 + rs.sym(ne, 0.2)).astype(np.float32), ffn_norm=(1.0 + rs.sym(ne, 0.2)).astype(np.float32))
        L["wq"] = make_tensor(rs, t["wq"], ne, nh * d)
        L["wk"] = make_tensor(rs, t["wk"], ne, nkv * d)
        L["wv"] = make_tensor(rs, t["wv"], ne, nkv * d)
        L["wo"] = make_tensor(rs, t["wo"], nh * d, ne)
        L["ffn_gate"] = make_tensor(rs, t["ffn_gate"], ne, nff)
        L["ffn_up"] = make_tensor(rs, t["ffn_up"], ne, nff)
        L["ffn_down"] = make_tensor(rs, t["ffn_down"], nff, ne)
        if c["bias"]:
            L["bq"], L["bk"], L["bv"] = rs.sym(nh * d, 0.3), rs.sym(nkv * d, 0.3), rs.sym(nkv * d, 0.3)
        if c["qk_norm"]:
            L["q_norm"] = (1.0 + rs.sym(d, 0.3)).astype(np.float32)
            L["k_norm"] = (1.0 + rs.sym(d, 0.3)).astype(np.float32)
        model["layers"].append(L)
    return model
