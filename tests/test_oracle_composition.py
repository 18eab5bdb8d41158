"""Pins the LAYER COMPOSITION of the stage oracle (oracle/stage.py: StageOracle.forward / _moe / logits) against a
decoder layer written separately, straight from the architecture definitions, in torch float64 with library
routines: F.rms_norm, F.scaled_dot_product_attention(enable_gqa, boolean causal mask), F.silu, torch.softmax /
torch.topk, complex-number rotation for RoPE.  The only thing shared with the oracle is `oracle.dequantize`, which
tests/test_oracle_formats.py pins on its own; none of oracle/stage.py is imported by the reference side.

What the architectures prescribe (ggml graph of one layer as rpc_server::graph_compute receives it,
third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451; tensor names
third_party/llama.cpp/patches/0003-moe-add-expert-analysis-and-split-tools.patch:945-955):
  h   = x + Wo . attention(rope(q), rope(k), v)        q, k, v = W{q,k,v} . rms_norm(x, attn_norm) (+ bias on qwen2)
  out = h + Wdown . (silu(Wgate . n) * (Wup . n))       n = rms_norm(h, ffn_norm)
  llama: neighbouring-pair rotation; qwen2 / qwen3: half-split (NEOX) rotation; qwen3: per-head rms_norm of q and k
  BEFORE the rotation; qwen3moe: softmax over all experts -> (+ 0 / -inf mask on the selection probabilities,
  patches/0003:86-104) -> top-k -> weights renormalised to sum 1 -> sum_e w_e * FFN_e(n).
The KV cache holds f16 (launch.rs:585-589), so K and V are rounded through torch.half before attention.

Each deliberately broken variant of the reference (a dropped residual, swapped norm weights, rotation before the
q/k norm, no renormalisation, ...) must be REJECTED by the same comparison: that is what shows the check can see
such a mistake in the oracle.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import models
import oracle
from oracle.stage import StageOracle

TOL = 1e-4          # relative L2 of what the layers add, f32-storing oracle against the float64 reference (measured: up to 3e-5)
BROKEN_MIN = 1e-2   # every broken variant must be at least this far away


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


def _model(name, seed=3, **kw):
    """The synthetic model, made SENSITIVE to its own structure: sigma-0.02 weights give q.k logits of ~0.1 (attention
    would be a plain average whatever the positions) and norm weights of 1 +- 0.02 commute with almost anything.  So
    the attention norm is scaled up until the softmax is peaked, and every norm gets clearly non-uniform weights."""
    cfg = models.CONFIGS[name]
    kvs, tl = models.build_tensors(cfg, range(cfg["n_layer"]), seed=seed, with_embd=True, with_output=True, **kw)
    tensors = {n: (t, d, x) for n, t, d, x in tl}
    rng = np.random.Generator(np.random.PCG64(seed + 1000))
    for n in list(tensors):
        if n.endswith("_norm.weight"):
            t, d, x = tensors[n]
            gain = 6.0 if n.endswith("attn_norm.weight") else 1.0
            f = (gain * rng.uniform(0.5, 2.0, x.size // 4)).astype(np.float32)
            tensors[n] = (t, d, (x.view(np.float32) * f).view(np.uint8))
        if n.endswith(".bias"):
            t, d, x = tensors[n]
            tensors[n] = (t, d, (x.view(np.float32) * 10).view(np.uint8))          # sigma 0.2 instead of 0.02
    return cfg, tensors


class TorchDecoder:
    """float64 decoder over dequantised weights; keeps the whole K / V history per sequence instead of a cache."""

    def __init__(self, cfg, tensors, expert_mask=None, broken=None):
        self.c, self.broken, self.mask = cfg, broken, expert_mask
        self.w = {}
        for name, (ttype, dims, data) in tensors.items():
            n = int(np.prod(dims))
            self.w[name] = torch.from_numpy(oracle.dequantize(ttype, data, n).astype(np.float64)).reshape(tuple(reversed(dims)))
        self.hist = {}      # (layer, seq) -> (K [n, HK, hd], V [n, HK, hd], positions)

    def _rope(self, x, pos):
        """x [T, H, hd]; rotation of pairs by pos * base^(-2i/hd) as a complex multiplication."""
        c = self.c
        hd = c["head_dim"]
        i = torch.arange(hd // 2, dtype=torch.float64)
        ang = torch.as_tensor(pos, dtype=torch.float64)[:, None] * c["rope"] ** (-2.0 * i / hd)
        rot = torch.polar(torch.ones_like(ang), ang)[:, None, :]                      # [T, 1, hd/2]
        if c["arch"] == "llama":
            z = torch.view_as_complex(x.reshape(*x.shape[:-1], hd // 2, 2).contiguous()) * rot
            return torch.view_as_real(z).reshape(x.shape)
        z = torch.complex(x[..., :hd // 2], x[..., hd // 2:]) * rot
        return torch.cat([z.real, z.imag], dim=-1)

    def _ffn(self, p, n):
        w, c = self.w, self.c
        if p + "ffn_gate.weight" in w:
            return (F.silu(n @ w[p + "ffn_gate.weight"].T) * (n @ w[p + "ffn_up.weight"].T)) @ w[p + "ffn_down.weight"].T
        probs = torch.softmax(n @ w[p + "ffn_gate_inp.weight"].T, dim=-1)
        sel = probs if self.mask is None else probs + torch.as_tensor(self.mask, dtype=torch.float64)
        ids = torch.topk(sel, c["n_expert_used"], dim=-1).indices
        wts = torch.gather(probs, 1, ids)
        if self.broken != "moe_no_renorm":
            wts = wts / wts.sum(dim=-1, keepdim=True)
        out = torch.zeros(n.shape[0], c["n_embd"], dtype=torch.float64)
        for t in range(n.shape[0]):
            for e, we in zip(ids[t].tolist(), wts[t]):
                g, u, d = w[p + "ffn_gate_exps.weight"][e], w[p + "ffn_up_exps.weight"][e], w[p + "ffn_down_exps.weight"][e]
                out[t] += we * ((F.silu(g @ n[t]) * (u @ n[t])) @ d.T)
        return out

    def forward(self, x, pos, seq, lb, le):
        c, w, br = self.c, self.w, self.broken
        x = torch.from_numpy(np.asarray(x, np.float64))
        T = x.shape[0]
        H, HK, hd, eps = c["n_head"], c["n_head_kv"], c["head_dim"], c["eps"]
        for il in range(lb, le):
            p = "blk.%d." % il
            an, fn = p + "attn_norm.weight", p + "ffn_norm.weight"
            if br == "swap_norm_weights":
                an, fn = fn, an
            n = F.rms_norm(x, (c["n_embd"],), w[an], eps)
            if br == "no_attn_norm":
                n = x
            q, k, v = n @ w[p + "attn_q.weight"].T, n @ w[p + "attn_k.weight"].T, n @ w[p + "attn_v.weight"].T
            if p + "attn_q.bias" in w and br != "no_bias":
                q, k, v = q + w[p + "attn_q.bias"], k + w[p + "attn_k.bias"], v + w[p + "attn_v.bias"]
            q, k, v = q.reshape(T, H, hd), k.reshape(T, HK, hd), v.reshape(T, HK, hd)
            qk_norm = p + "attn_q_norm.weight" in w
            if qk_norm and br != "rope_before_qk_norm":
                q, k = F.rms_norm(q, (hd,), w[p + "attn_q_norm.weight"], eps), F.rms_norm(k, (hd,), w[p + "attn_k_norm.weight"], eps)
            if br != "no_rope":
                q, k = self._rope(q, pos), self._rope(k, pos)
            if br == "rope_v":
                v = self._rope(v, pos)
            if qk_norm and br == "rope_before_qk_norm":
                q, k = F.rms_norm(q, (hd,), w[p + "attn_q_norm.weight"], eps), F.rms_norm(k, (hd,), w[p + "attn_k_norm.weight"], eps)
            k, v = k.half().double(), v.half().double()          # the cache rows are f16
            att = torch.empty(T, H, hd, dtype=torch.float64)
            for t in range(T):
                key = (il, int(seq[t]))
                K0, V0, P0 = self.hist.get(key, (k[:0], v[:0], []))
                # a position written again replaces the cached row
                keep = [i for i, pp in enumerate(P0) if pp != int(pos[t])]
                K1, V1 = torch.cat([K0[keep], k[t:t + 1]]), torch.cat([V0[keep], v[t:t + 1]])
                P1 = [P0[i] for i in keep] + [int(pos[t])]
                self.hist[key] = (K1, V1, P1)
                visible = torch.tensor([pp <= int(pos[t]) for pp in P1])
                scale = None if br != "no_attn_scale" else 1.0
                o = F.scaled_dot_product_attention(q[t][None, :, None, :], K1.transpose(0, 1)[None], V1.transpose(0, 1)[None],
                                                   attn_mask=visible[None, None, None, :], enable_gqa=True, scale=scale)
                att[t] = o[0, :, 0, :]
            h = att.reshape(T, H * hd) @ w[p + "attn_output.weight"].T
            x = h if br == "no_attn_residual" else x + h
            n = F.rms_norm(x, (c["n_embd"],), w[fn], eps)
            f = self._ffn(p, n)
            x = f if br == "no_ffn_residual" else x + f
        return x.numpy()

    def logits(self, x):
        w, c = self.w, self.c
        n = F.rms_norm(torch.from_numpy(np.asarray(x, np.float64)), (c["n_embd"],), w["output_norm.weight"], c["eps"])
        out = w["output.weight"] if "output.weight" in w else w["token_embd.weight"]
        return (n @ out.T).numpy()


def _walk(cfg, tensors, ref, lb, le, mask=None):
    """Prefill of two sequences, single-token steps, a mixed batch and an overwrite of a cached position: the oracle's
    outputs and the reference's, call by call."""
    orc = StageOracle(cfg, tensors, lb, le, 32, n_seq_max=2, expert_mask=mask)
    rng = np.random.Generator(np.random.PCG64(17))
    E = cfg["n_embd"]
    outs = []
    calls = [(np.arange(7), np.zeros(7, int)), (np.arange(3), np.ones(3, int)), ([7], [0]), ([8], [0]), ([3, 9, 4, 10], [1, 0, 1, 0]), ([2], [1])]
    for pos, seq in calls:
        x = (3.0 * rng.standard_normal((len(pos), E))).astype(np.float32)      # not unit RMS: the norms have something to do
        # what the layers ADD to the hidden state is compared (the residual stream itself would hide it)
        outs.append((orc.forward(x, pos, seq=seq) - x, ref.forward(x, pos, seq, lb, le) - x))
    return outs, orc


ARCHS = ["tiny-llama", "tiny-qwen2", "tiny-qwen3", "tiny-moe", "tiny-g5"]


@pytest.mark.parametrize("name", ARCHS)
def test_stage_oracle_equals_independent_float64_decoder(name):
    cfg, tensors = _model(name)
    nl = cfg["n_layer"]
    lb = 1 if nl > 2 else 0
    outs, orc = _walk(cfg, tensors, TorchDecoder(cfg, tensors), lb, nl)
    for i, (got, want) in enumerate(outs):
        assert rel_l2(got, want) <= TOL, (name, i, rel_l2(got, want))
    # output head of the last stage
    x = 3.0 * np.random.Generator(np.random.PCG64(2)).standard_normal((3, cfg["n_embd"])).astype(np.float32)
    assert rel_l2(orc.logits(x), TorchDecoder(cfg, tensors).logits(x)) <= TOL


def test_moe_mask_and_shard_follow_the_reference_definition():
    """Expert mask: 0 / -inf added to the selection probabilities before top-k (patches/0003:86-104), the mixing weights
    still come from the unmasked softmax and are renormalised over the selected experts."""
    cfg, tensors = _model("tiny-moe")
    allowed = np.zeros(cfg["n_expert"], bool)
    allowed[[0, 3, 5, 6]] = True
    mask = np.where(allowed, 0.0, -np.inf).astype(np.float32)
    outs, orc = _walk(cfg, tensors, TorchDecoder(cfg, tensors, expert_mask=mask), 0, cfg["n_layer"], mask=mask)
    for got, want in outs:
        assert rel_l2(got, want) <= TOL
    assert set(np.concatenate(orc.last_expert_ids).tolist()) <= {0, 3, 5, 6}
    # and the mask matters: the unmasked reference is far from the masked oracle
    outs_nomask, _ = _walk(cfg, tensors, TorchDecoder(cfg, tensors), 0, cfg["n_layer"], mask=mask)
    assert max(rel_l2(g, w) for g, w in outs_nomask) > BROKEN_MIN


BROKEN = [("tiny-llama", "no_attn_residual"), ("tiny-llama", "no_ffn_residual"), ("tiny-llama", "swap_norm_weights"),
          ("tiny-llama", "no_attn_norm"), ("tiny-llama", "no_rope"), ("tiny-llama", "rope_v"), ("tiny-llama", "no_attn_scale"),
          ("tiny-qwen2", "no_bias"), ("tiny-qwen3", "rope_before_qk_norm"), ("tiny-moe", "moe_no_renorm")]


@pytest.mark.parametrize("name,broken", BROKEN)
def test_comparison_rejects_broken_compositions(name, broken):
    cfg, tensors = _model(name)
    nl = cfg["n_layer"]
    lb = 1 if nl > 2 else 0
    # the intact reference still agrees on exactly these tensors ...
    good, _ = _walk(cfg, tensors, TorchDecoder(cfg, tensors), lb, nl)
    assert max(rel_l2(g, w) for g, w in good) <= TOL
    # ... and the broken one does not
    bad, _ = _walk(cfg, tensors, TorchDecoder(cfg, tensors, broken=broken), lb, nl)
    assert max(rel_l2(g, w) for g, w in bad) > BROKEN_MIN, (name, broken, max(rel_l2(g, w) for g, w in bad))
