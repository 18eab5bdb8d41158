"""CPU oracle of a pipeline stage: the per-layer graph a mesh-llm worker executes for its layer range
(rpc_server::graph_compute, third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451),
composed from the pinned primitives of mesh_oracle.c.

TEST INFRASTRUCTURE ONLY.  Parity against llama.cpp's CPU backend is unpinned: activations stay f32 and
accumulate in f64 here, where ggml rounds them to Q8_K blocks before an integer dot and keeps some f16
intermediates in flash attention.  What is pinned: every primitive (tests/test_oracle_ops.py); the layer
composition (forward, _moe, logits) against a decoder written separately in torch float64 from the architecture
definitions, which must also reject deliberately broken compositions (tests/test_oracle_composition.py); and
its invariants (prefill == token-by-token decode, batch invariance, stage split == unsplit model;
tests/test_oracle_stage.py).
"""
import numpy as np

import oracle as O


class StageOracle:
    """tensors: dict name -> (ggml_type, dims (ne0, ne1[, ne2]), uint8 ndarray) as written to the GGUF file."""

    def __init__(self, cfg, tensors, layer_begin, layer_end, n_ctx, n_seq_max=1, expert_mask=None, kv_types=None, blas=False):
        """blas: projections of calls with many tokens go through numpy's float64 matmul over the dequantised matrix
        (x @ dequantize(W).T -- the definition mesh_oracle.c's mul_mat is pinned to in tests/test_oracle_ops.py) instead
        of the C loop, which keeps prefill-sized checks within seconds.
        kv_types: (K type, V type) of the cache, each F16, Q8_0 or Q4_0 (the tiers of
        mesh-llm/src/inference/launch.rs:568-591); None = f16 / f16.  A quantised cache is held as the f32 values its
        blocks dequantise to (rows quantised per 32 elements along head_dim, as ggml stores the cache rows)."""
        self.c = cfg
        self.t = tensors
        self.lb, self.le = layer_begin, layer_end
        self.n_ctx = n_ctx
        hk, hd = cfg["n_head_kv"], cfg["head_dim"]
        self.kv_types = tuple(kv_types) if kv_types else (O.F16, O.F16)
        self.kv_f32 = self.kv_types != (O.F16, O.F16)
        self.k = np.zeros((layer_end - layer_begin, n_seq_max, hk, n_ctx, hd), np.float32 if self.kv_f32 else np.uint16)
        self.v = np.zeros_like(self.k)
        self.rope_mode = O.ROPE_NORM if cfg["arch"] == "llama" else O.ROPE_NEOX
        self.expert_mask = expert_mask
        self.blas = blas

    def _w(self, name):
        ttype, dims, data = self.t[name]
        return ttype, dims, data

    def _f32(self, name):
        ttype, dims, data = self.t[name]
        assert ttype == O.F32
        return data.view(np.float32)

    def _mm(self, name, x, bias=None):
        ttype, dims, data = self._w(name)
        K, M = dims[0], dims[1]
        b = self._f32(bias) if bias is not None and bias in self.t else None
        if self.blas and x.shape[0] >= 32:
            x64 = np.asarray(x, np.float64)
            y = np.empty((x.shape[0], M), np.float32)
            rb = O.row_bytes(ttype, K)
            for m0 in range(0, M, 1024):          # row blocks: the float64 copy of a block stays cache-sized
                m1 = min(M, m0 + 1024)
                Wd = O.dequantize(ttype, data[m0 * rb:m1 * rb], (m1 - m0) * K).reshape(m1 - m0, K).astype(np.float64)
                blk = x64 @ Wd.T
                if b is not None:
                    blk += b[m0:m1].astype(np.float64)
                y[:, m0:m1] = blk
            return y
        return O.mul_mat(ttype, data, M, K, x, b)

    def embed(self, ids):
        ttype, dims, data = self._w("token_embd.weight")
        rb = O.row_bytes(ttype, dims[0])
        return np.stack([O.dequantize(ttype, data[i * rb:(i + 1) * rb], dims[0]) for i in ids])

    def logits(self, x):
        n = O.rms_norm(x, self._f32("output_norm.weight"), self.c["eps"])
        name = "output.weight" if "output.weight" in self.t else "token_embd.weight"
        return self._mm(name, n)

    def _head_norm(self, x, wname):
        """qwen3 per-head RMS norm over head_dim: x [T, H, hd]."""
        T, H, hd = x.shape
        return O.rms_norm(x.reshape(T * H, hd), self._f32(wname), self.c["eps"]).reshape(T, H, hd)

    def _moe(self, p, n):
        c = self.c
        gi_t, gi_dims, gi = self._w(p + "ffn_gate_inp.weight")
        n_exp = gi_dims[1]
        logits = O.mul_mat(gi_t, gi, n_exp, gi_dims[0], n)
        T = n.shape[0]
        out = np.zeros((T, c["n_embd"]), np.float64)
        gt, gd, gdata = self._w(p + "ffn_gate_exps.weight")
        ut, ud, udata = self._w(p + "ffn_up_exps.weight")
        dt, dd, ddata = self._w(p + "ffn_down_exps.weight")
        FE, E = gd[1], gd[0]
        g_sz, d_sz = FE * O.row_bytes(gt, E), E * O.row_bytes(dt, FE)
        u_sz = FE * O.row_bytes(ut, E)
        self.last_expert_ids = []
        for t in range(T):
            ids, w = O.moe_route(logits[t], self.expert_mask, c["n_expert_used"], True)
            self.last_expert_ids.append(ids)
            for e, we in zip(ids, w):
                g = O.mul_mat(gt, gdata[e * g_sz:(e + 1) * g_sz], FE, E, n[t:t + 1])
                u = O.mul_mat(ut, udata[e * u_sz:(e + 1) * u_sz], FE, E, n[t:t + 1])
                h = O.swiglu(g, u)
                out[t] += float(we) * O.mul_mat(dt, ddata[e * d_sz:(e + 1) * d_sz], E, FE, h)[0].astype(np.float64)
        return out.astype(np.float32)

    def forward(self, x, pos, seq=None, kv_rows=None):
        """x: [T, n_embd] f32 -> [T, n_embd] f32 after layers [lb, le); updates the KV cache.
        kv_rows: {local layer index: (k [T, n_head_kv, head_dim] f32, v likewise)}: rows to put into the cache for this
        call's tokens in place of the ones computed here.  A test hands in the rows the device under test wrote, which
        separates its attention arithmetic from the sensitivity of a 4-bit cache quantiser to rounding upstream of it
        (a value near a decision threshold lands on the neighbouring code)."""
        c = self.c
        x = np.array(x, dtype=np.float32).reshape(-1, c["n_embd"])
        T = x.shape[0]
        pos = np.asarray(pos, np.int32)
        seq = np.zeros(T, np.int32) if seq is None else np.asarray(seq, np.int32)
        H, HK, hd = c["n_head"], c["n_head_kv"], c["head_dim"]
        scale = 1.0 / np.sqrt(hd)
        for il in range(self.lb, self.le):
            p = "blk.%d." % il
            li = il - self.lb
            n = O.rms_norm(x, self._f32(p + "attn_norm.weight"), c["eps"])
            q = self._mm(p + "attn_q.weight", n, p + "attn_q.bias").reshape(T, H, hd)
            k = self._mm(p + "attn_k.weight", n, p + "attn_k.bias").reshape(T, HK, hd)
            v = self._mm(p + "attn_v.weight", n, p + "attn_v.bias").reshape(T, HK, hd)
            if p + "attn_q_norm.weight" in self.t:
                q = self._head_norm(q, p + "attn_q_norm.weight")
                k = self._head_norm(k, p + "attn_k_norm.weight")
            q = O.rope(q, pos, hd, c["rope"], self.rope_mode)
            k = O.rope(k, pos, hd, c["rope"], self.rope_mode)
            if self.kv_f32:
                kh, vh = O.kv_round(self.kv_types[0], k), O.kv_round(self.kv_types[1], v)
            else:
                kh, vh = O.fp32_to_fp16(k), O.fp32_to_fp16(v)
            if kv_rows is not None and li in kv_rows:
                kh, vh = (np.asarray(r, np.float32).reshape(T, HK, hd) for r in kv_rows[li])
                if not self.kv_f32:
                    kh, vh = O.fp32_to_fp16(kh).reshape(T, HK, hd), O.fp32_to_fp16(vh).reshape(T, HK, hd)
            for t in range(T):
                self.k[li, seq[t], :, pos[t], :] = kh[t]
                self.v[li, seq[t], :, pos[t], :] = vh[t]
            att = np.empty((T, H, hd), np.float32)
            for t in range(T):
                att[t] = O.attn_token(q[t], self.k[li, seq[t]], self.v[li, seq[t]], int(pos[t]), scale)
            x = x + self._mm(p + "attn_output.weight", att.reshape(T, H * hd))
            n = O.rms_norm(x, self._f32(p + "ffn_norm.weight"), c["eps"])
            if p + "ffn_gate.weight" in self.t:
                h = O.swiglu(self._mm(p + "ffn_gate.weight", n), self._mm(p + "ffn_up.weight", n))
                x = x + self._mm(p + "ffn_down.weight", h)
            else:
                x = x + self._moe(p, n)
        return x
