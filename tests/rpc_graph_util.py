"""Serialized ggml graphs for the GRAPH_COMPUTE tests: the decoder sub-graph llama.cpp's graph builder emits for a range of
layers, as the RPC backend puts it on the wire (| device u32 | n_nodes u32 | node ids u64[] | n_tensors u32 | rpc_tensor[] |,
third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451,1070-1085).

llama.cpp is not vendored in the reference, so the node structure below is written from the published graph builder
(norm -> q/k/v -> rope -> cache store -> flash attention -> output projection -> residual -> norm -> gate/up -> swiglu ->
down -> residual, with the names the builder gives them) and the op numbers come from the server's own table
(mesh-llm_amd/csrc/rpc/ggml_ops.hpp, itself marked unverifiable).  The server recognises a graph by its weight names and
the shapes around them, so these graphs exercise what it relies on: leaves named like GGUF tensors, one f32 hidden-state
leaf, an `inp_pos` leaf, cache leaves, and the last node as the result."""
import os
import re
import struct

from rpc_client import TENSOR_FMT

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32, F16, Q4_0, Q8_0, I32, I64 = 0, 1, 2, 8, 26, 27
BLOCK = {0: (1, 4), 1: (1, 2), 2: (32, 18), 6: (32, 22), 8: (32, 34), 12: (256, 144), 14: (256, 210), 26: (1, 4), 27: (1, 8)}


def op_ids():
    text = open(os.path.join(ROOT, "mesh-llm_amd", "csrc", "rpc", "ggml_ops.hpp")).read()
    body = text[text.index("names[] = {"):text.index("};", text.index("names[] = {"))]
    return {n: i for i, n in enumerate(re.findall(r'"([A-Z0-9_]+)"', body))}


OP = op_ids()


def strides(ttype, ne):
    be, bb = BLOCK[ttype]
    nb = [bb, bb * (ne[0] // be)]
    nb.append(nb[1] * ne[1])
    nb.append(nb[2] * ne[2])
    return nb


class GraphBuilder:
    """Collects tensor descriptors; ids are made up like client-side addresses."""

    def __init__(self, buffer, base, device=0):
        self.buffer, self.at, self.device = buffer, base, device
        self.tensors, self.nodes, self.next_id = {}, [], 0x7F0000001000

    def _add(self, name, ttype, ne, op, srcs, view_src, view_offs, data):
        ne = list(ne) + [1] * (4 - len(ne))
        tid = self.next_id
        self.next_id += 0x150
        srcs = list(srcs) + [0] * (10 - len(srcs))
        self.tensors[tid] = struct.pack(TENSOR_FMT, tid, ttype, self.buffer, *ne, *strides(ttype, ne), op, *([0] * 16), 0, *srcs, view_src, view_offs, data,
                                        name.encode()[:63], b"")
        return tid

    def nbytes(self, ttype, ne):
        ne = list(ne) + [1] * (4 - len(ne))
        return strides(ttype, ne)[3] * ne[3]

    def leaf(self, name, ttype, ne):
        data = self.at
        self.at += (self.nbytes(ttype, ne) + 255) // 256 * 256
        return self._add(name, ttype, ne, 0, [], 0, 0, data)

    def node(self, name, op, ne, srcs, ttype=F32, view_of=None):
        if view_of is not None:
            tid = self._add(name, ttype, ne, OP[op], srcs, view_of, 0, self.data_of(view_of))
        else:
            data = self.at
            self.at += (self.nbytes(ttype, ne) + 255) // 256 * 256
            tid = self._add(name, ttype, ne, OP[op], srcs, 0, 0, data)
        self.nodes.append(tid)
        return tid

    def descriptor(self, tid):
        return self.tensors[tid]

    def data_of(self, tid):
        return struct.unpack(TENSOR_FMT, self.tensors[tid])[-3]

    def payload(self, nodes=None, drop=()):
        nodes = self.nodes if nodes is None else nodes
        ts = [t for tid, t in self.tensors.items() if tid not in drop]
        return struct.pack("<II", self.device, len(nodes)) + b"".join(struct.pack("<Q", n) for n in nodes) + struct.pack("<I", len(ts)) + b"".join(ts)


def layer_range_graph(gb, weights, layers, T, n_head, n_head_kv, head_dim, n_ctx, cache_types=(F16, F16), with_output=False, backend="RPC0[127.0.0.1:50052]"):
    """weights: {gguf name: (type, dims)}.  Returns ids of the hidden-state input, the positions and the result."""
    E = weights["blk.%d.attn_norm.weight" % layers[0]][1][0]
    w = {name: gb.leaf(name, t, dims) for name, (t, dims) in weights.items()}
    inp = gb.leaf("%s#l_out-%d#0" % (backend, layers[0] - 1) if layers[0] else "%s#inp_embd#0" % backend, F32, [E, T])
    pos = gb.leaf("%s#inp_pos#0" % backend, I32, [T])
    mask = gb.leaf("%s#KQ_mask#0" % backend, F16, [n_ctx, (T + 63) // 64 * 64])
    kd = n_head_kv * head_dim
    cur = inp
    for il in layers:
        p = "blk.%d." % il
        ck = gb.leaf("cache_k_l%d" % il, cache_types[0], [kd, n_ctx])
        cv = gb.leaf("cache_v_l%d" % il, cache_types[1], [kd, n_ctx])
        norm = gb.node("norm-%d" % il, "RMS_NORM", [E, T], [cur])
        an = gb.node("attn_norm-%d" % il, "MUL", [E, T], [norm, w[p + "attn_norm.weight"]])
        q = gb.node("Qcur-%d" % il, "MUL_MAT", [n_head * head_dim, T], [w[p + "attn_q.weight"], an])
        k = gb.node("Kcur-%d" % il, "MUL_MAT", [kd, T], [w[p + "attn_k.weight"], an])
        v = gb.node("Vcur-%d" % il, "MUL_MAT", [kd, T], [w[p + "attn_v.weight"], an])
        for nm, t_, rows in (("q", q, n_head * head_dim), ("k", k, kd), ("v", v, kd)):
            if p + "attn_%s.bias" % nm in w:
                t2 = gb.node("%scur-%d" % (nm.upper(), il), "ADD", [rows, T], [t_, w[p + "attn_%s.bias" % nm]])
                q, k, v = (t2 if nm == "q" else q), (t2 if nm == "k" else k), (t2 if nm == "v" else v)
        q3 = gb.node("Qcur-%d (reshaped)" % il, "RESHAPE", [head_dim, n_head, T], [q], view_of=q)
        k3 = gb.node("Kcur-%d (reshaped)" % il, "RESHAPE", [head_dim, n_head_kv, T], [k], view_of=k)
        if p + "attn_q_norm.weight" in w:
            qn = gb.node("norm-%d" % il, "RMS_NORM", [head_dim, n_head, T], [q3])
            q3 = gb.node("Qcur_normed-%d" % il, "MUL", [head_dim, n_head, T], [qn, w[p + "attn_q_norm.weight"]])
            kn = gb.node("norm-%d" % il, "RMS_NORM", [head_dim, n_head_kv, T], [k3])
            k3 = gb.node("Kcur_normed-%d" % il, "MUL", [head_dim, n_head_kv, T], [kn, w[p + "attn_k_norm.weight"]])
        qr = gb.node("Qcur-%d" % il, "ROPE", [head_dim, n_head, T], [q3, pos])
        kr = gb.node("Kcur-%d" % il, "ROPE", [head_dim, n_head_kv, T], [k3, pos])
        kv_ = gb.node("k_cache_view-%d" % il, "VIEW", [kd, T], [ck], ttype=cache_types[0], view_of=ck)
        gb.node("k_cache_view-%d (copy of Kcur-%d)" % (il, il), "CPY", [kd, T], [kr, kv_], ttype=cache_types[0], view_of=kv_)
        vv_ = gb.node("v_cache_view-%d" % il, "VIEW", [kd, T], [cv], ttype=cache_types[1], view_of=cv)
        gb.node("v_cache_view-%d (copy of Vcur-%d)" % (il, il), "CPY", [kd, T], [v, vv_], ttype=cache_types[1], view_of=vv_)
        qp = gb.node("q-%d" % il, "PERMUTE", [head_dim, T, n_head], [qr], view_of=qr)
        kk = gb.node("k-%d" % il, "VIEW", [head_dim, n_ctx, n_head_kv], [ck], ttype=cache_types[0], view_of=ck)
        vk = gb.node("v-%d" % il, "VIEW", [head_dim, n_ctx, n_head_kv], [cv], ttype=cache_types[1], view_of=cv)
        fa = gb.node("__fattn__-%d" % il, "FLASH_ATTN_EXT", [head_dim, n_head, T], [qp, kk, vk, mask])
        kqv = gb.node("kqv_out-%d" % il, "RESHAPE", [n_head * head_dim, T], [fa], view_of=fa)
        ao = gb.node("attn_out-%d" % il, "MUL_MAT", [E, T], [w[p + "attn_output.weight"], kqv])
        ffn_inp = gb.node("ffn_inp-%d" % il, "ADD", [E, T], [ao, cur])
        norm2 = gb.node("norm-%d" % il, "RMS_NORM", [E, T], [ffn_inp])
        fn = gb.node("ffn_norm-%d" % il, "MUL", [E, T], [norm2, w[p + "ffn_norm.weight"]])
        if p + "ffn_gate.weight" in w:
            FF = weights[p + "ffn_gate.weight"][1][1]
            g_ = gb.node("ffn_gate-%d" % il, "MUL_MAT", [FF, T], [w[p + "ffn_gate.weight"], fn])
            u_ = gb.node("ffn_up-%d" % il, "MUL_MAT", [FF, T], [w[p + "ffn_up.weight"], fn])
            sw = gb.node("ffn_swiglu-%d" % il, "GLU", [FF, T], [g_, u_])
            out = gb.node("ffn_out-%d" % il, "MUL_MAT", [E, T], [w[p + "ffn_down.weight"], sw])
        else:
            n_exp, n_used = weights[p + "ffn_gate_inp.weight"][1][1], 2
            FE = weights[p + "ffn_gate_exps.weight"][1][1]
            logits = gb.node("ffn_moe_logits-%d" % il, "MUL_MAT", [n_exp, T], [w[p + "ffn_gate_inp.weight"], fn])
            probs = gb.node("ffn_moe_probs-%d" % il, "SOFT_MAX", [n_exp, T], [logits])
            sel = gb.node("ffn_moe_topk-%d" % il, "ARGSORT", [n_used, T], [probs], ttype=I32)
            up = gb.node("ffn_moe_up-%d" % il, "MUL_MAT_ID", [FE, n_used, T], [w[p + "ffn_up_exps.weight"], fn, sel])
            ga = gb.node("ffn_moe_gate-%d" % il, "MUL_MAT_ID", [FE, n_used, T], [w[p + "ffn_gate_exps.weight"], fn, sel])
            sw = gb.node("ffn_moe_swiglu-%d" % il, "GLU", [FE, n_used, T], [ga, up])
            dn = gb.node("ffn_moe_down-%d" % il, "MUL_MAT_ID", [E, n_used, T], [w[p + "ffn_down_exps.weight"], sw, sel])
            out = gb.node("ffn_moe_out-%d" % il, "ADD", [E, T], [dn, dn])
        cur = gb.node("l_out-%d" % il, "ADD", [E, T], [out, ffn_inp])
    if with_output:
        rn = gb.node("norm", "RMS_NORM", [E, T], [cur])
        on = gb.node("result_norm", "MUL", [E, T], [rn, w["output_norm.weight"]])
        ow = "output.weight" if "output.weight" in w else "token_embd.weight"
        cur = gb.node("result_output", "MUL_MAT", [weights[ow][1][1], T], [w[ow], on])
    return inp, pos, cur
