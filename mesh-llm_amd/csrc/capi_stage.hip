// extern "C" entry points for weights, GGUF inspection and the stage executor (include/mesh_stage.h).

#include <cmath>
#include <cstring>
#include <vector>

#include "gemv.hpp"
#include "attn.hpp"
#include "stage.hpp"

struct mesh_weight {
    mesh::DevTensor t;
    size_t gguf_bytes = 0;
};

using namespace mesh;

extern "C" {

int mesh_weight_upload(int type, const void *host_data, int64_t n_rows, int64_t row_len, mesh_weight **out) {
    if (!host_data || !out || n_rows <= 0 || row_len <= 0) return fail(MESH_ERR_INVALID, "mesh_weight_upload: null pointer or empty shape");
    *out = nullptr;
    const int64_t rb = row_bytes(type, row_len);
    if (rb < 0) return fail(block_elems(type) < 0 ? MESH_ERR_UNSUPPORTED : MESH_ERR_INVALID,
                            "mesh_weight_upload: row length %lld is not a whole number of type-%d blocks", (long long)row_len, type);
    mesh_weight *w = new mesh_weight();
    w->t.type = type; w->t.K = row_len; w->t.M = n_rows; w->t.E = 1;
    w->gguf_bytes = (size_t)(rb * n_rows);
    w->t.tiled = type_is_tiled(type);
    w->t.bytes = w->t.tiled ? (size_t)tiled_bytes(type, n_rows, row_len) : w->gguf_bytes;
    hipError_t e = hipMalloc(&w->t.data, w->t.bytes);
    if (e != hipSuccess) {
        const size_t wanted = w->t.bytes;
        delete w;
        return fail(MESH_ERR_NOMEM, "mesh_weight_upload: hipMalloc(%zu) failed: %s", wanted, hipGetErrorString(e));
    }
    int rc = MESH_OK;
    if (!w->t.tiled) {
        e = hipMemcpy(w->t.data, host_data, w->gguf_bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) rc = fail(MESH_ERR_DEVICE, "mesh_weight_upload: copy failed: %s", hipGetErrorString(e));
    } else {
        void *tmp = nullptr;
        e = hipMalloc(&tmp, w->gguf_bytes);
        if (e != hipSuccess) rc = fail(MESH_ERR_NOMEM, "mesh_weight_upload: hipMalloc(%zu) failed", w->gguf_bytes);
        if (rc == MESH_OK && (e = hipMemcpy(tmp, host_data, w->gguf_bytes, hipMemcpyHostToDevice)) != hipSuccess)
            rc = fail(MESH_ERR_DEVICE, "mesh_weight_upload: copy failed: %s", hipGetErrorString(e));
        if (rc == MESH_OK) rc = repack_tiled(type, tmp, w->t.data, n_rows, row_len, nullptr);
        if (rc == MESH_OK && (e = hipDeviceSynchronize()) != hipSuccess)
            rc = fail(MESH_ERR_DEVICE, "mesh_weight_upload: repack failed: %s", hipGetErrorString(e));
        if (tmp) (void)hipFree(tmp);
    }
    if (rc != MESH_OK) { (void)hipFree(w->t.data); delete w; return rc; }
    *out = w;
    return MESH_OK;
}

void mesh_weight_free(mesh_weight *w) {
    if (!w) return;
    if (w->t.data) (void)hipFree(w->t.data);
    delete w;
}

size_t mesh_weight_nbytes(const mesh_weight *w) { return w ? w->gguf_bytes : 0; }

int mesh_weight_download(const mesh_weight *w, void *host_data) {
    if (!w || !host_data) return fail(MESH_ERR_INVALID, "mesh_weight_download: null argument");
    if (!w->t.tiled) {
        MESH_HIP_TRY(hipMemcpy(host_data, w->t.data, w->gguf_bytes, hipMemcpyDeviceToHost));
        return MESH_OK;
    }
    void *tmp = nullptr;
    MESH_HIP_TRY(hipMalloc(&tmp, w->gguf_bytes));
    int rc = unpack_tiled(w->t.type, w->t.data, tmp, w->t.M, w->t.K, nullptr);
    if (rc == MESH_OK && hipMemcpy(host_data, tmp, w->gguf_bytes, hipMemcpyDeviceToHost) != hipSuccess)
        rc = fail(MESH_ERR_DEVICE, "mesh_weight_download: copy failed");
    (void)hipFree(tmp);
    return rc;
}

int mesh_mul_mat_dev(const mesh_weight *w, const float *d_x, int64_t n_tokens, float *d_y, void *stream) {
    if (!w || !d_x || !d_y || n_tokens < 0) return fail(MESH_ERR_INVALID, "mesh_mul_mat_dev: null argument");
    if (n_tokens == 0) return MESH_OK;
    GemvArgs a;
    a.n_mat = 1;
    a.mat[0].W = w->t.data; a.mat[0].type = w->t.type; a.mat[0].M = (int)w->t.M; a.mat[0].y = d_y; a.mat[0].ldy = (int)w->t.M;
    a.x = d_x; a.ldx = (int)w->t.K; a.K = (int)w->t.K; a.T = (int)n_tokens;
    return gemv(a, static_cast<hipStream_t>(stream));
}

static void fill_info(const HParams &hp, mesh_model_info *o) {
    memset(o, 0, sizeof *o);
    strncpy(o->arch, hp.arch.c_str(), sizeof(o->arch) - 1);
    o->n_layer = hp.n_layer; o->n_embd = hp.n_embd; o->n_head = hp.n_head; o->n_head_kv = hp.n_head_kv;
    o->head_dim = hp.head_dim; o->n_ff = hp.n_ff; o->n_vocab = hp.n_vocab; o->n_rot = hp.n_rot; o->rope_mode = hp.rope_mode;
    o->n_expert = hp.n_expert; o->n_expert_used = hp.n_expert_used; o->n_ff_exp = hp.n_ff_exp;
    o->rms_eps = hp.rms_eps; o->rope_freq_base = hp.rope_freq_base;
}

int mesh_gguf_probe(const char *gguf_path, mesh_model_info *out) {
    if (!out) return fail(MESH_ERR_INVALID, "mesh_gguf_probe: null output");
    GgufFile g;
    int rc = g.open(gguf_path);
    if (rc != MESH_OK) return rc;
    HParams hp;
    if ((rc = hparams_from_gguf(g, hp)) != MESH_OK) return rc;
    fill_info(hp, out);
    out->gguf_version = g.version(); out->alignment = g.alignment();
    out->n_tensors = g.tensors().size(); out->data_offset = g.data_offset(); out->file_size = g.file_size();
    return MESH_OK;
}

int mesh_gguf_tensor(const char *gguf_path, const char *name, mesh_tensor_info *out) {
    if (!name || !out) return fail(MESH_ERR_INVALID, "mesh_gguf_tensor: null argument");
    GgufFile g;
    int rc = g.open(gguf_path);
    if (rc != MESH_OK) return rc;
    const GgufTensorInfo *t = g.find(name);
    if (!t) return fail(MESH_ERR_INVALID, "mesh_gguf_tensor: tensor '%s' not found", name);
    memset(out, 0, sizeof *out);
    out->type = t->type; out->n_dims = t->n_dims;
    for (int i = 0; i < 4; ++i) out->ne[i] = t->ne[i];
    out->file_offset = g.data_offset() + t->offset;
    out->nbytes = t->nbytes;
    if (t->nbytes == 0) return fail(MESH_ERR_UNSUPPORTED, "mesh_gguf_tensor: tensor '%s' has ggml type %u, unknown to this build", name, t->type);
    if (!g.data(*t)) return fail(MESH_ERR_FORMAT, "mesh_gguf_tensor: tensor '%s' (%llu bytes at %llu) lies outside the file", name,
                                 (unsigned long long)t->nbytes, (unsigned long long)out->file_offset);
    return MESH_OK;
}

int mesh_stage_open(const char *gguf_path, int layer_begin, int layer_end, const mesh_stage_opts *opts, mesh_stage **out) {
    return stage_open(gguf_path, layer_begin, layer_end, opts, out);
}

void mesh_stage_close(mesh_stage *stage) { delete stage; }

int mesh_stage_info(const mesh_stage *stage, mesh_model_info *out) {
    if (!stage || !out) return fail(MESH_ERR_INVALID, "mesh_stage_info: null argument");
    fill_info(stage->hp, out);
    return MESH_OK;
}

size_t mesh_stage_weight_bytes(const mesh_stage *stage) { return stage ? stage->weight_bytes : 0; }

int mesh_stage_session_new(mesh_stage *stage, mesh_session **out) { return session_new(stage, out); }

void mesh_stage_session_free(mesh_session *session) { delete session; }

int mesh_stage_decode(mesh_session *session, const mesh_batch *batch, const void *in, int in_fmt, void *out, int out_fmt,
                      size_t out_cap, size_t *out_len) {
    return stage_decode(session, batch, in, in_fmt, out, out_fmt, out_cap, out_len);
}

int mesh_stage_decode_dev(mesh_session *session, const mesh_batch *batch, const void *d_in, int in_fmt, void *d_out,
                          int out_fmt, size_t out_cap, size_t *out_len) {
    return stage_decode_dev(session, batch, d_in, in_fmt, d_out, out_fmt, out_cap, out_len);
}

void *mesh_session_stream(mesh_session *session) { return session ? static_cast<void *>(session->stream) : nullptr; }

int mesh_session_synchronize(mesh_session *session) {
    if (!session) return fail(MESH_ERR_INVALID, "mesh_session_synchronize: null session");
    MESH_HIP_TRY(hipStreamSynchronize(session->stream));
    return MESH_OK;
}

int64_t mesh_session_graph_replays(const mesh_session *session) {
    return session ? session->graph_replays : -1;
}

int mesh_session_profile(mesh_session *session, int enable) {
    if (!session) return fail(MESH_ERR_INVALID, "mesh_session_profile: null session");
    int rc = profile_collect(session);
    if (rc != MESH_OK) return rc;
    session->profile = enable != 0;
    for (int i = 0; i < MESH_PROF_KINDS; ++i) { session->prof_ms[i] = 0; session->prof_launches[i] = 0; }
    return MESH_OK;
}

int mesh_session_profile_read(mesh_session *session, mesh_profile *out) {
    if (!session || !out) return fail(MESH_ERR_INVALID, "mesh_session_profile_read: null argument");
    int rc = profile_collect(session);
    if (rc != MESH_OK) return rc;
    for (int i = 0; i < MESH_PROF_KINDS; ++i) { out->ms[i] = session->prof_ms[i]; out->launches[i] = session->prof_launches[i]; }
    return MESH_OK;
}

int mesh_session_set_expert_mask(mesh_session *session, const uint8_t *allowed, int32_t n_mask) {
    if (!session) return fail(MESH_ERR_INVALID, "mesh_session_set_expert_mask: null session");
    const mesh_stage *st = session->stage;
    if (!session->expert_mask) return fail(MESH_ERR_INVALID, "mesh_session_set_expert_mask: the stage has no mixture-of-experts layers");
    if (!allowed) { session->expert_mask_on = false; return MESH_OK; }
    const int ne = (int)st->layers[0].gate_inp.M;
    if (n_mask != ne) return fail(MESH_ERR_INVALID, "mesh_session_set_expert_mask: mask has %d entries, the file holds %d experts", n_mask, ne);
    std::vector<float> m((size_t)ne);
    for (int e = 0; e < ne; ++e) m[(size_t)e] = allowed[e] ? 0.0f : -INFINITY;
    MESH_HIP_TRY(hipSetDevice(st->device));
    MESH_HIP_TRY(hipStreamSynchronize(session->stream));
    MESH_HIP_TRY(hipMemcpy(session->expert_mask, m.data(), m.size() * sizeof(float), hipMemcpyHostToDevice));
    session->expert_mask_on = true;
    return MESH_OK;
}

int mesh_session_moe_last_ids(mesh_session *session, int32_t *ids, int32_t n_tokens) {
    if (!session || !ids || !session->moe_ids) return fail(MESH_ERR_INVALID, "mesh_session_moe_last_ids: no mixture-of-experts state");
    const mesh_stage *st = session->stage;
    if (n_tokens <= 0 || n_tokens > st->n_batch_max) return fail(MESH_ERR_INVALID, "mesh_session_moe_last_ids: bad token count");
    MESH_HIP_TRY(hipStreamSynchronize(session->stream));
    MESH_HIP_TRY(hipMemcpy(ids, session->moe_ids, (size_t)n_tokens * st->hp.n_expert_used * sizeof(int32_t), hipMemcpyDeviceToHost));
    return MESH_OK;
}

int mesh_session_f16_saturations(mesh_session *session, uint64_t *count) {
    if (!session || !count) return fail(MESH_ERR_INVALID, "mesh_session_f16_saturations: null argument");
    unsigned v = 0;
    MESH_HIP_TRY(hipSetDevice(session->stage->device));
    MESH_HIP_TRY(hipStreamSynchronize(session->stream));
    MESH_HIP_TRY(hipMemcpy(&v, session->f16_sat, sizeof(v), hipMemcpyDeviceToHost));
    // the device counter is 32 bits wide and wraps; the host keeps the running total
    session->f16_sat_total += (uint32_t)(v - session->f16_sat_seen);
    session->f16_sat_seen = v;
    *count = session->f16_sat_total;
    return MESH_OK;
}

int mesh_session_set_option(mesh_session *session, const char *name, int32_t value) {
    if (!session || !name) return fail(MESH_ERR_INVALID, "mesh_session_set_option: null argument");
    Tuning t = session->tune;
    const int rc = tuning_set(t, name, value, true);
    if (rc != MESH_OK) return rc;
    // launches captured under the old value would replay it
    MESH_HIP_TRY(hipSetDevice(session->stage->device));
    MESH_HIP_TRY(hipStreamSynchronize(session->stream));
    for (auto &g : session->graphs)
        if (g.second.exec) (void)hipGraphExecDestroy(g.second.exec);
    session->graphs.clear();
    session->tune = t;
    return MESH_OK;
}

int mesh_session_get_option(const mesh_session *session, const char *name, int32_t *value) {
    if (!session || !name || !value) return fail(MESH_ERR_INVALID, "mesh_session_get_option: null argument");
    int v = 0;
    const int rc = tuning_get(session->tune, name, &v);
    if (rc == MESH_OK) *value = v;
    return rc;
}

static int kv_xfer(mesh_session *s, int layer, int seq_id, int pos0, int n_pos, uint16_t *k, uint16_t *v, bool write) {
    if (!s || !k || !v) return fail(MESH_ERR_INVALID, "mesh_session_kv: null argument");
    const mesh_stage *st = s->stage;
    const HParams &hp = st->hp;
    if (layer < st->layer_begin || layer >= st->layer_end) return fail(MESH_ERR_INVALID, "mesh_session_kv: layer %d not in this stage [%d,%d)", layer, st->layer_begin, st->layer_end);
    if (seq_id < 0 || seq_id >= st->n_seq_max || pos0 < 0 || n_pos <= 0 || pos0 + n_pos > st->n_ctx)
        return fail(MESH_ERR_INVALID, "mesh_session_kv: sequence %d positions [%d,%d) outside the cache", seq_id, pos0, pos0 + n_pos);
    MESH_HIP_TRY(hipSetDevice(st->device));
    MESH_HIP_TRY(hipStreamSynchronize(s->stream));
    // through a device buffer of f16 rows [n_pos][n_head_kv][head_dim]: the cache rows may be quantised
    const int hd = (int)hp.head_dim, nkv = (int)hp.n_head_kv;
    const size_t bytes = (size_t)n_pos * nkv * hd * 2;
    uint16_t *tmp = nullptr;
    MESH_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&tmp), bytes));
    int rc = MESH_OK;
    for (int which = 0; which < 2 && rc == MESH_OK; ++which) {
        const size_t lb = which ? s->v_layer_bytes : s->k_layer_bytes;
        uint8_t *cache = (which ? s->vcache : s->kcache) + (size_t)(layer - st->layer_begin) * lb;
        const int type = which ? st->v_type : st->k_type;
        uint16_t *host = which ? v : k;
        hipError_t e = hipSuccess;
        if (write) {
            e = hipMemcpyAsync(tmp, host, bytes, hipMemcpyHostToDevice, s->stream);
            if (e == hipSuccess) rc = kv_import(type, cache, tmp, nkv, st->n_ctx, hd, seq_id, pos0, n_pos, s->stream);
        } else {
            rc = kv_export(type, cache, tmp, nkv, st->n_ctx, hd, seq_id, pos0, n_pos, s->stream);
            if (rc == MESH_OK) e = hipMemcpyAsync(host, tmp, bytes, hipMemcpyDeviceToHost, s->stream);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
        if (e != hipSuccess && rc == MESH_OK) rc = fail(MESH_ERR_DEVICE, "mesh_session_kv: %s", hipGetErrorString(e));
    }
    (void)hipFree(tmp);
    return rc;
}

int mesh_session_kv_write(mesh_session *session, int layer, int seq_id, int pos0, int n_pos, const uint16_t *k, const uint16_t *v) {
    return kv_xfer(session, layer, seq_id, pos0, n_pos, const_cast<uint16_t *>(k), const_cast<uint16_t *>(v), true);
}

int mesh_session_kv_read(mesh_session *session, int layer, int seq_id, int pos0, int n_pos, uint16_t *k, uint16_t *v) {
    return kv_xfer(session, layer, seq_id, pos0, n_pos, k, v, false);
}

}  // extern "C"
