// `mesh-stage-plugin`: the stage as a mesh-llm plugin process that provides an inference endpoint.
//
// The plugin host (mesh-llm/src/plugin/runtime.rs) spawns the executable with MESH_LLM_PLUGIN_ENDPOINT naming a unix
// socket; both sides exchange frames of a u32 little-endian length followed by a protobuf Envelope, at most 16 MiB
// (mesh-llm/plugin/src/io.rs:118-184, protocol version 2: plugin/src/lib.rs:78).  The host sends InitializeRequest and
// expects an InitializeResponse that repeats the plugin's configured name and protocol version and carries the manifest
// (runtime.rs:237-290); an endpoint of kind INFERENCE over HTTP with protocol "openai_compatible" is then probed with
// GET <address>/models, whose {"data":[{"id":..}]} ids become the models the mesh routes here (src/plugin/mod.rs:1614-1711),
// and HealthRequest / ShutdownRequest follow the same request-id discipline.  `managed_by_plugin` marks the endpoint as
// one this process owns (what `inference::provider` sets, plugin/src/dsl.rs:469-476).
//
// What the endpoint serves: /v1/models (the stage's model id), and POST /v1/stage/decode, the stage's own operation --
// packed boundary activations in, packed boundary activations (or logits) out.  Chat / completion routes answer 501: a
// pipeline stage has no tokenizer and no sampler, those stay with the process that owns both ends of the pipeline.

#include <algorithm>
#include <arpa/inet.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <sys/socket.h>
#include <sys/un.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../../include/mesh_stage.h"
#include "pb_wire.hpp"

namespace mesh_plugin {

constexpr uint32_t PROTOCOL_VERSION = 2;
constexpr size_t MAX_FRAME = 16u * 1024 * 1024;
// Envelope: protocol_version = 1, plugin_id = 2, request_id = 3, payload oneof:
constexpr uint32_t ENV_INITIALIZE_REQUEST = 10, ENV_INITIALIZE_RESPONSE = 11, ENV_HEALTH_REQUEST = 12, ENV_HEALTH_RESPONSE = 13,
                   ENV_SHUTDOWN_REQUEST = 14, ENV_SHUTDOWN_RESPONSE = 15, ENV_ERROR_RESPONSE = 20;
constexpr int32_t ERR_METHOD_NOT_FOUND = -32601;        // JSON-RPC's code, as the SDK's PluginError::method_not_found uses
constexpr uint64_t ENDPOINT_KIND_INFERENCE = 1, ENDPOINT_TRANSPORT_HTTP = 1, HEALTH_STATUS_OK = 1, HEALTH_STATUS_UNHEALTHY = 3;

struct Config {
    std::string plugin_id = "mesh-stage";
    std::string gguf;
    int layer_begin = 0, layer_end = -1;
    std::string device;
    int n_ctx = 4096, n_seq_max = 1, n_batch_max = 512;
    bool open_stage = true;          // --no-stage: serve /v1/models from the file's header only (machines without a GPU)
    int http_port = 0;               // 0 = any free port
};

struct State {
    Config cfg;
    mesh_model_info info{};
    std::string model_id;
    mesh_stage *stage = nullptr;
    mesh_session *session = nullptr;
    std::mutex decode_mu;            // one session, one caller at a time
    int http_fd = -1, http_port = 0;
    std::atomic<bool> stopping{false};
};

static bool write_all(int fd, const void *p, size_t n) {
    const char *c = static_cast<const char *>(p);
    while (n) {
        const ssize_t k = ::send(fd, c, n, MSG_NOSIGNAL);
        if (k < 0 && errno == EINTR) continue;
        if (k <= 0) return false;
        c += k;
        n -= (size_t)k;
    }
    return true;
}
static bool read_all(int fd, void *p, size_t n) {
    char *c = static_cast<char *>(p);
    while (n) {
        const ssize_t k = ::recv(fd, c, n, 0);
        if (k < 0 && errno == EINTR) continue;
        if (k <= 0) return false;
        c += k;
        n -= (size_t)k;
    }
    return true;
}

static std::string json_escape(const std::string &s) {
    std::string o;
    for (unsigned char ch : s) {
        if (ch == '"' || ch == '\\') { o += '\\'; o += (char)ch; }
        else if (ch < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", ch); o += b; }
        else o += (char)ch;
    }
    return o;
}

// ---- envelopes ------------------------------------------------------------------------------------------------------
static bool send_envelope(int fd, const State &st, uint64_t request_id, uint32_t payload_field, const std::string &payload) {
    PbWriter env;
    env.u64(1, PROTOCOL_VERSION);
    env.str(2, st.cfg.plugin_id);
    env.u64(3, request_id);
    env.bytes(payload_field, payload);
    const std::string &body = env.data();
    const uint32_t len = (uint32_t)body.size();
    return write_all(fd, &len, 4) && write_all(fd, body.data(), body.size());
}

static std::string endpoint_address(const State &st) { return "http://127.0.0.1:" + std::to_string(st.http_port) + "/v1"; }

static std::string initialize_response(const State &st) {
    // EndpointManifest: endpoint_id 1, kind 2, transport_kind 3, protocol 4, address 5, supports_streaming 8, managed_by_plugin 9
    PbWriter ep;
    ep.str(1, "stage");
    ep.u64(2, ENDPOINT_KIND_INFERENCE);
    ep.u64(3, ENDPOINT_TRANSPORT_HTTP);
    ep.bytes(4, "openai_compatible");
    ep.bytes(5, endpoint_address(st));
    ep.boolean(8, false);
    ep.boolean(9, true);
    // PluginManifest: endpoints 7, capabilities 8
    PbWriter mf;
    mf.bytes(7, ep.data());
    mf.str(8, "mesh.stage.v1");
    // InitializeResponse: plugin_id 1, plugin_protocol_version 2, plugin_version 3, server_info_json 4, capabilities 5, manifest 6
    PbWriter r;
    r.str(1, st.cfg.plugin_id);
    r.u64(2, PROTOCOL_VERSION);
    r.str(3, "0.2.0");
    char info[512];
    snprintf(info, sizeof info, "{\"model\":\"%s\",\"arch\":\"%s\",\"layers\":[%d,%d],\"n_embd\":%u,\"stage_open\":%s}", json_escape(st.model_id).c_str(), st.info.arch,
             st.cfg.layer_begin, st.cfg.layer_end < 0 ? (int)st.info.n_layer : st.cfg.layer_end, st.info.n_embd, st.session ? "true" : "false");
    r.str(4, info);
    r.str(5, "mesh.stage.v1");
    r.bytes(6, mf.data());
    return r.data();
}

static int serve_host(int fd, State &st) {
    for (;;) {
        uint32_t len = 0;
        if (!read_all(fd, &len, 4)) return 0;                      // host went away: exit quietly
        if (len > MAX_FRAME) {
            fprintf(stderr, "[mesh-stage-plugin] frame of %u bytes exceeds the 16 MiB limit\n", len);
            return 1;
        }
        std::string body(len, '\0');
        if (len && !read_all(fd, &body[0], len)) return 0;
        PbReader env(body);
        uint64_t request_id = 0;
        uint32_t payload_field = 0;
        while (env.next()) {
            if (env.field == 3 && env.wire == 0) request_id = env.value;
            else if (env.field >= 10 && env.wire == 2) payload_field = env.field;
        }
        if (!env.ok()) {
            fprintf(stderr, "[mesh-stage-plugin] malformed envelope\n");
            return 1;
        }
        switch (payload_field) {
            case ENV_INITIALIZE_REQUEST:
                if (!send_envelope(fd, st, request_id, ENV_INITIALIZE_RESPONSE, initialize_response(st))) return 0;
                break;
            case ENV_HEALTH_REQUEST: {
                PbWriter h;                                        // HealthResponse: status 1, detail 2
                const bool ok = st.session != nullptr || !st.cfg.open_stage;
                h.u64(1, ok ? HEALTH_STATUS_OK : HEALTH_STATUS_UNHEALTHY);
                h.str(2, st.session ? "stage open, endpoint " + endpoint_address(st) : "model listed, stage not opened");
                if (!send_envelope(fd, st, request_id, ENV_HEALTH_RESPONSE, h.data())) return 0;
                break;
            }
            case ENV_SHUTDOWN_REQUEST:
                (void)send_envelope(fd, st, request_id, ENV_SHUTDOWN_RESPONSE, "");
                return 0;
            case 0:
                break;                                             // an envelope without a payload: nothing to answer
            default: {
                if (request_id == 0) break;                        // notifications and events need no reply
                PbWriter e;                                        // ErrorResponse: code 1 (int32 as varint), message 2
                e.u64(1, (uint64_t)(int64_t)ERR_METHOD_NOT_FOUND);
                e.str(2, "mesh-stage-plugin does not handle payload " + std::to_string(payload_field));
                if (!send_envelope(fd, st, request_id, ENV_ERROR_RESPONSE, e.data())) return 0;
            }
        }
    }
}

// ---- HTTP endpoint --------------------------------------------------------------------------------------------------
static void http_reply(int fd, const char *status, const char *ctype, const std::string &body) {
    char head[256];
    const int n = snprintf(head, sizeof head, "HTTP/1.1 %s\r\nContent-Type: %s\r\nContent-Length: %zu\r\nConnection: close\r\n\r\n", status, ctype, body.size());
    if (write_all(fd, head, (size_t)n)) (void)write_all(fd, body.data(), body.size());
}
static void http_error(int fd, const char *status, const std::string &message, const char *type) {
    http_reply(fd, status, "application/json", "{\"error\":{\"message\":\"" + json_escape(message) + "\",\"type\":\"" + type + "\"}}");
}

static std::string header_value(const std::string &head, const char *name) {
    // case-insensitive search for "\r\nname:"
    const std::string needle = std::string("\r\n") + name + ":";
    for (size_t i = 0; i + needle.size() <= head.size(); ++i) {
        if (strncasecmp(head.data() + i, needle.data(), needle.size()) == 0) {
            size_t a = i + needle.size();
            while (a < head.size() && head[a] == ' ') ++a;
            const size_t b = head.find("\r\n", a);
            return head.substr(a, b == std::string::npos ? std::string::npos : b - a);
        }
    }
    return "";
}

static int format_id(const std::string &name, int fallback) {
    if (name == "f32") return MESH_F32;
    if (name == "f16") return MESH_F16;
    if (name == "q8_0") return MESH_Q8_0;
    if (name == "tokens") return MESH_TOKENS;
    if (name == "logits") return MESH_LOGITS;
    return name.empty() ? fallback : -1;
}

// POST /v1/stage/decode: headers X-Mesh-Tokens (count), X-Mesh-Pos0 (cache position of the first token; the rest follow),
// X-Mesh-Seq (sequence id, default 0), X-Mesh-In-Format / X-Mesh-Out-Format (f32 | f16 | q8_0, in also tokens, out also
// logits; default q8_0); body = the packed input rows.  200 with the packed output rows as application/octet-stream.
static void handle_decode(int fd, State &st, const std::string &head, const std::string &body) {
    if (!st.session) return http_error(fd, "503 Service Unavailable", "the stage is not open in this process", "stage_unavailable");
    const int T = atoi(header_value(head, "X-Mesh-Tokens").c_str());
    const int pos0 = atoi(header_value(head, "X-Mesh-Pos0").c_str());
    const int seq = atoi(header_value(head, "X-Mesh-Seq").c_str());
    const int in_fmt = format_id(header_value(head, "X-Mesh-In-Format"), MESH_Q8_0), out_fmt = format_id(header_value(head, "X-Mesh-Out-Format"), MESH_Q8_0);
    if (T < 1 || T > st.cfg.n_batch_max || pos0 < 0 || pos0 > (1 << 30) || seq < 0 || in_fmt < 0 || out_fmt < 0 || in_fmt == MESH_LOGITS || out_fmt == MESH_TOKENS)
        return http_error(fd, "400 Bad Request", "X-Mesh-Tokens / X-Mesh-Pos0 / formats out of range", "invalid_request_error");
    // (refused before anything is allocated for it: a row of logits is the whole vocabulary)
    if (out_fmt == MESH_LOGITS && T > MESH_LOGITS_TOKENS_MAX)
        return http_error(fd, "400 Bad Request", "logits of at most " + std::to_string(MESH_LOGITS_TOKENS_MAX) + " tokens per request", "invalid_request_error");
    const size_t want = in_fmt == MESH_TOKENS ? (size_t)T * 4 : mesh_act_packed_size(in_fmt, T, st.info.n_embd);
    if (body.size() != want) return http_error(fd, "400 Bad Request", "body has " + std::to_string(body.size()) + " bytes, " + std::to_string(want) + " expected", "invalid_request_error");
    std::vector<int32_t> pos((size_t)T), seqs((size_t)T, seq);
    for (int i = 0; i < T; ++i) pos[(size_t)i] = pos0 + i;
    mesh_batch b{T, pos.data(), seqs.data()};
    const size_t cap = out_fmt == MESH_LOGITS ? (size_t)T * st.info.n_vocab * 4 : mesh_act_packed_size(out_fmt, T, st.info.n_embd);
    std::string out(cap, '\0');
    size_t len = 0;
    int rc;
    {
        std::lock_guard<std::mutex> lk(st.decode_mu);
        if (st.stopping || !st.session) return http_error(fd, "503 Service Unavailable", "the plugin is shutting down", "stage_unavailable");
        rc = mesh_stage_decode(st.session, &b, body.data(), in_fmt, &out[0], out_fmt, cap, &len);
    }
    if (rc != MESH_OK) return http_error(fd, rc == MESH_ERR_INVALID ? "400 Bad Request" : "500 Internal Server Error", mesh_last_error(), "stage_error");
    out.resize(len);
    http_reply(fd, "200 OK", "application/octet-stream", out);
}

static void http_client(int fd, State *st) {
    std::string req;
    char buf[65536];
    size_t head_end = std::string::npos;
    while (head_end == std::string::npos && req.size() < (1u << 20)) {
        const ssize_t n = ::recv(fd, buf, sizeof buf, 0);
        if (n <= 0) { ::close(fd); return; }
        req.append(buf, (size_t)n);
        head_end = req.find("\r\n\r\n");
    }
    if (head_end == std::string::npos) { ::close(fd); return; }
    const std::string head = req.substr(0, head_end + 2);
    const size_t clen = (size_t)strtoull(header_value(head, "Content-Length").c_str(), nullptr, 10);
    std::string body = req.substr(head_end + 4);
    // (the largest body a stage takes is a batch of f32 rows)
    const size_t body_max = std::max<size_t>(1u << 20, st->session ? (size_t)st->cfg.n_batch_max * st->info.n_embd * 4 : 0);
    if (clen > body_max) { http_error(fd, "413 Payload Too Large", "body too large", "invalid_request_error"); ::close(fd); return; }
    while (body.size() < clen) {
        const ssize_t n = ::recv(fd, buf, sizeof buf, 0);
        if (n <= 0) break;
        body.append(buf, (size_t)n);
    }
    const size_t sp1 = head.find(' '), sp2 = head.find(' ', sp1 + 1);
    const std::string method = head.substr(0, sp1);
    std::string path = sp1 == std::string::npos || sp2 == std::string::npos ? "" : head.substr(sp1 + 1, sp2 - sp1 - 1);
    const size_t q = path.find('?');
    if (q != std::string::npos) path.resize(q);
    if (method == "GET" && (path == "/v1/models" || path == "/models")) {
        http_reply(fd, "200 OK", "application/json", "{\"object\":\"list\",\"data\":[{\"id\":\"" + json_escape(st->model_id) + "\",\"object\":\"model\",\"owned_by\":\"mesh-stage\"}]}");
    } else if (method == "POST" && path == "/v1/stage/decode") {
        if (body.size() != clen) http_error(fd, "400 Bad Request", "truncated body", "invalid_request_error");
        else handle_decode(fd, *st, head, body);
    } else if (method == "POST" && (path == "/v1/chat/completions" || path == "/v1/completions" || path == "/v1/responses" || path == "/v1/embeddings")) {
        http_error(fd, "501 Not Implemented", "this endpoint serves a pipeline stage (POST /v1/stage/decode); tokenisation and sampling belong to the process that owns both ends of the pipeline", "not_implemented");
    } else {
        http_error(fd, "404 Not Found", "no such route", "invalid_request_error");
    }
    ::shutdown(fd, SHUT_RDWR);
    ::close(fd);
}

static bool http_listen(State &st) {
    const int fd = ::socket(AF_INET, SOCK_STREAM, 0);
    if (fd < 0) return false;
    int one = 1;
    (void)setsockopt(fd, SOL_SOCKET, SO_REUSEADDR, &one, sizeof one);
    sockaddr_in addr{};
    addr.sin_family = AF_INET;
    addr.sin_addr.s_addr = htonl(INADDR_LOOPBACK);
    addr.sin_port = htons((uint16_t)st.cfg.http_port);
    socklen_t len = sizeof addr;
    if (::bind(fd, reinterpret_cast<sockaddr *>(&addr), sizeof addr) != 0 || ::listen(fd, 64) != 0 ||
        getsockname(fd, reinterpret_cast<sockaddr *>(&addr), &len) != 0) {
        ::close(fd);
        return false;
    }
    st.http_fd = fd;
    st.http_port = ntohs(addr.sin_port);
    std::thread([&st]() {
        while (!st.stopping) {
            const int c = ::accept(st.http_fd, nullptr, nullptr);
            if (c < 0) {
                if (st.stopping) break;
                continue;
            }
            std::thread(http_client, c, &st).detach();
        }
    }).detach();
    return true;
}

static std::string model_id_of(const std::string &path) {
    size_t a = path.find_last_of('/');
    std::string base = a == std::string::npos ? path : path.substr(a + 1);
    if (base.size() > 5 && base.compare(base.size() - 5, 5, ".gguf") == 0) base.resize(base.size() - 5);
    return base;
}

}  // namespace mesh_plugin

int main(int argc, char **argv) {
    using namespace mesh_plugin;
    State st;
    Config &c = st.cfg;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        auto val = [&]() -> const char * { return i + 1 < argc ? argv[++i] : ""; };
        if (a == "--plugin-id") c.plugin_id = val();
        else if (a == "--gguf" || a == "-m") c.gguf = val();
        else if (a == "--layers") {                                 // BEGIN:END, END exclusive, empty = to the last layer
            const std::string v = val();
            const size_t colon = v.find(':');
            c.layer_begin = atoi(v.c_str());
            c.layer_end = colon == std::string::npos || colon + 1 >= v.size() ? -1 : atoi(v.c_str() + colon + 1);
        } else if (a == "-d" || a == "--device") c.device = val();
        else if (a == "-c" || a == "--ctx-size") c.n_ctx = atoi(val());
        else if (a == "--parallel") c.n_seq_max = atoi(val());
        else if (a == "--batch") c.n_batch_max = atoi(val());
        else if (a == "--http-port") c.http_port = atoi(val());
        else if (a == "--no-stage") c.open_stage = false;
        else {
            fprintf(stderr, "usage: %s --gguf PATH [--layers B:E] [-d ROCm0] [-c CTX] [--parallel N] [--batch N] [--plugin-id NAME] [--http-port P] [--no-stage]\n", argv[0]);
            return 2;
        }
    }
    if (const char *id = getenv("MESH_LLM_PLUGIN_NAME")) if (*id) c.plugin_id = id;      // the name the host configured (src/plugin/runtime.rs:188) and checks the reply against
    if (c.gguf.empty()) { fprintf(stderr, "[mesh-stage-plugin] --gguf is required\n"); return 2; }
    if (mesh_gguf_probe(c.gguf.c_str(), &st.info) != MESH_OK) { fprintf(stderr, "[mesh-stage-plugin] %s\n", mesh_last_error()); return 1; }
    st.model_id = model_id_of(c.gguf);
    signal(SIGPIPE, SIG_IGN);
    if (c.open_stage) {
        mesh_stage_opts o{};
        o.device = c.device.empty() ? nullptr : c.device.c_str();
        o.n_ctx = c.n_ctx; o.n_seq_max = c.n_seq_max; o.n_batch_max = c.n_batch_max;
        if (mesh_stage_open(c.gguf.c_str(), c.layer_begin, c.layer_end, &o, &st.stage) != MESH_OK ||
            mesh_stage_session_new(st.stage, &st.session) != MESH_OK) {
            fprintf(stderr, "[mesh-stage-plugin] cannot open the stage: %s\n", mesh_last_error());
            return 1;
        }
    }
    if (!http_listen(st)) { fprintf(stderr, "[mesh-stage-plugin] cannot listen on 127.0.0.1\n"); return 1; }
    const char *endpoint = getenv("MESH_LLM_PLUGIN_ENDPOINT");
    const char *transport = getenv("MESH_LLM_PLUGIN_TRANSPORT");
    if (!endpoint || !*endpoint) { fprintf(stderr, "[mesh-stage-plugin] MESH_LLM_PLUGIN_ENDPOINT is not set for plugin process\n"); return 1; }
    if (transport && *transport && strcmp(transport, "unix") != 0) { fprintf(stderr, "[mesh-stage-plugin] Unsupported plugin transport '%s'\n", transport); return 1; }
    const int fd = ::socket(AF_UNIX, SOCK_STREAM, 0);
    sockaddr_un sa{};
    sa.sun_family = AF_UNIX;
    strncpy(sa.sun_path, endpoint, sizeof sa.sun_path - 1);
    if (fd < 0 || ::connect(fd, reinterpret_cast<sockaddr *>(&sa), sizeof sa) != 0) {
        fprintf(stderr, "[mesh-stage-plugin] cannot connect to %s: %s\n", endpoint, strerror(errno));
        return 1;
    }
    const int rc = serve_host(fd, st);
    st.stopping = true;
    ::close(fd);
    if (st.http_fd >= 0) { ::shutdown(st.http_fd, SHUT_RDWR); ::close(st.http_fd); }
    {
        // a request thread may be inside a decode call: wait for it, and let later ones find the session gone
        std::lock_guard<std::mutex> lk(st.decode_mu);
        if (st.session) mesh_stage_session_free(st.session);
        st.session = nullptr;
        if (st.stage) mesh_stage_close(st.stage);
        st.stage = nullptr;
    }
    return rc;
}
