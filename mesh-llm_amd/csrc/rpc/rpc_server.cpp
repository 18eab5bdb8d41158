// Command loop of the rpc-server-compatible front end.  Behaviour follows rpc_serve_client / rpc_server of the reference
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch: peer registry :472-500, staged push
// :544-622, per-connection thread and shared server state :1927-1935,2309-2329, PEER_TENSOR_DATA = SET_TENSOR with a
// result byte :2233-2246; patches/0001-rpc-optimize-local-GGUF-tensor-loading.patch:179-266 for SET_TENSOR_GGUF): a
// request that fails validation ends the connection, a command with a result byte reports 0 instead.

#include "rpc_server.hpp"

#include <algorithm>
#include <arpa/inet.h>
#include <netdb.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <sys/socket.h>
#include <unistd.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <fstream>
#include <thread>

#include "../../../include/mesh_stage.h"

namespace mesh_rpc {

// ------------------------------------------------------------------------------------------------ byte stream
Conn::~Conn() {
    if (fd_ >= 0) ::close(fd_);
}

bool Conn::send_all(const void *data, size_t size) {
    const char *p = static_cast<const char *>(data);
    while (size > 0) {
        const ssize_t n = ::send(fd_, p, size, MSG_NOSIGNAL);
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) return false;
        p += n;
        size -= (size_t)n;
    }
    return true;
}

bool Conn::recv_all(void *data, size_t size) {
    char *p = static_cast<char *>(data);
    while (size > 0) {
        const ssize_t n = ::recv(fd_, p, size, 0);
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) return false;
        p += n;
        size -= (size_t)n;
    }
    return true;
}

bool Conn::send_msg(const void *data, uint64_t size) {
    return send_all(&size, sizeof size) && (size == 0 || send_all(data, size));
}

bool Conn::recv_msg(void *data, uint64_t size) {
    uint64_t got = 0;
    if (!recv_all(&got, sizeof got) || got != size) return false;
    return size == 0 || recv_all(data, size);
}

bool Conn::recv_msg(std::vector<uint8_t> &data, uint64_t limit) {
    uint64_t size = 0;
    if (!recv_all(&size, sizeof size) || size > limit) return false;
    try {
        data.resize(size);
    } catch (const std::exception &) {
        return false;
    }
    return size == 0 || recv_all(data.data(), size);
}

static void tune_socket(int fd) {
    int one = 1;
    (void)setsockopt(fd, IPPROTO_TCP, TCP_NODELAY, &one, sizeof one);
}

std::unique_ptr<Conn> Conn::connect_to(const std::string &host, int port) {
    addrinfo hints{};
    hints.ai_family = AF_INET;
    hints.ai_socktype = SOCK_STREAM;
    addrinfo *res = nullptr;
    if (getaddrinfo(host.c_str(), std::to_string(port).c_str(), &hints, &res) != 0 || !res) return nullptr;
    const int fd = ::socket(res->ai_family, res->ai_socktype, res->ai_protocol);
    if (fd < 0 || ::connect(fd, res->ai_addr, res->ai_addrlen) != 0) {
        if (fd >= 0) ::close(fd);
        freeaddrinfo(res);
        return nullptr;
    }
    freeaddrinfo(res);
    tune_socket(fd);
    return std::unique_ptr<Conn>(new Conn(fd));
}

// ------------------------------------------------------------------------------------------------ server
Server::Server(BufferBackend *backend, ServerConfig cfg) : backend_(backend), cfg_(std::move(cfg)) {}

Server::~Server() {
    stop();
    std::lock_guard<std::mutex> lk(mu_);
    for (auto &kv : buffers_) backend_->release(kv.second->dev, kv.second->base);
    buffers_.clear();
}

void Server::log(const char *fmt, ...) {
    char buf[640];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    fprintf(stderr, "[rpc-server] %s\n", buf);
    fflush(stderr);
}

void Server::debug(const char *fmt, ...) {
    if (!cfg_.verbose) return;
    char buf[640];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    fprintf(stderr, "[rpc-server] %s\n", buf);
    fflush(stderr);
}

int Server::listen_on() {
    const int fd = ::socket(AF_INET, SOCK_STREAM, 0);
    if (fd < 0) return -1;
    int one = 1;
    (void)setsockopt(fd, SOL_SOCKET, SO_REUSEADDR, &one, sizeof one);
    sockaddr_in addr{};
    addr.sin_family = AF_INET;
    addr.sin_port = htons((uint16_t)cfg_.port);
    if (inet_pton(AF_INET, cfg_.host.c_str(), &addr.sin_addr) != 1) {
        log("cannot parse host '%s' (an IPv4 address is expected)", cfg_.host.c_str());
        ::close(fd);
        return -1;
    }
    if (::bind(fd, reinterpret_cast<sockaddr *>(&addr), sizeof addr) != 0 || ::listen(fd, 64) != 0) {
        log("cannot listen on %s:%d: %s", cfg_.host.c_str(), cfg_.port, strerror(errno));
        ::close(fd);
        return -1;
    }
    socklen_t len = sizeof addr;
    if (getsockname(fd, reinterpret_cast<sockaddr *>(&addr), &len) == 0) cfg_.port = ntohs(addr.sin_port);
    listen_fd_ = fd;
    return cfg_.port;
}

void Server::stop() {
    const int fd = listen_fd_.exchange(-1);
    if (fd >= 0) {
        ::shutdown(fd, SHUT_RDWR);
        ::close(fd);
    }
    std::unique_lock<std::mutex> lk(clients_mu_);
    for (int cfd : client_fds_) ::shutdown(cfd, SHUT_RDWR);       // their blocking reads return; the threads close the sockets themselves
    clients_cv_.wait_for(lk, std::chrono::seconds(10), [this]() { return client_fds_.empty(); });
}

void Server::serve() {
    for (;;) {
        const int lfd = listen_fd_.load();
        if (lfd < 0) break;
        const int fd = ::accept(lfd, nullptr, nullptr);
        if (fd < 0) {
            if (listen_fd_.load() < 0) break;
            if (errno == EINTR || errno == ECONNABORTED) continue;
            log("accept failed: %s", strerror(errno));
            break;
        }
        tune_socket(fd);
        printf("Accepted client connection\n");
        fflush(stdout);
        {
            std::lock_guard<std::mutex> lk(clients_mu_);
            client_fds_.insert(fd);
        }
        std::thread([this, fd]() {
            {
                Conn conn(fd);
                serve_client(conn);
                printf("Client connection closed\n");
                fflush(stdout);
                std::lock_guard<std::mutex> lk(clients_mu_);      // (before the socket closes: the number cannot be reused while it is listed)
                client_fds_.erase(fd);
                clients_cv_.notify_all();                         // under the lock: the last thing this thread does with the server
            }
        }).detach();
    }
}

const Server::Buffer *Server::locate(const Tensor &t, uint64_t offset, uint64_t size, const char *what) {
    auto it = buffers_.find(t.buffer);
    if (t.buffer == 0 || it == buffers_.end()) {
        log("%s: tensor '%.64s' names no live buffer", what, t.name);
        return nullptr;
    }
    const Buffer *b = it->second.get();
    const uint64_t p0 = (uint64_t)(uintptr_t)b->base, p1 = p0 + b->size;
    const uint64_t nbytes = tensor_nbytes(t);
    if (nbytes == 0 || t.data < p0 || t.data > p1 || nbytes > p1 - t.data) {
        log("%s: tensor '%.64s' (type %u, %llu bytes at 0x%llx) does not lie inside its buffer [0x%llx, 0x%llx)", what, t.name, t.type,
            (unsigned long long)nbytes, (unsigned long long)t.data, (unsigned long long)p0, (unsigned long long)p1);
        return nullptr;
    }
    if (offset > nbytes || size > nbytes - offset) {
        log("%s: range offset %llu size %llu leaves tensor '%.64s' of %llu bytes", what, (unsigned long long)offset, (unsigned long long)size,
            t.name, (unsigned long long)nbytes);
        return nullptr;
    }
    return b;
}

bool Server::set_tensor(const std::vector<uint8_t> &input) {
    if (input.size() < sizeof(Tensor) + sizeof(uint64_t)) return false;
    Tensor t;
    uint64_t offset;
    memcpy(&t, input.data(), sizeof t);
    memcpy(&offset, input.data() + sizeof t, sizeof offset);
    const uint64_t size = input.size() - sizeof t - sizeof offset;
    std::lock_guard<std::mutex> lk(mu_);
    const Buffer *b = locate(t, offset, size, "set_tensor");
    if (!b) return false;
    debug("set_tensor '%.64s' offset %llu size %llu", t.name, (unsigned long long)offset, (unsigned long long)size);
    return size == 0 || backend_->upload(b->dev, reinterpret_cast<void *>((uintptr_t)(t.data + offset)), input.data() + sizeof t + sizeof offset, size);
}

bool Server::get_tensor(const GetTensorReq &req, std::vector<uint8_t> &out) {
    std::lock_guard<std::mutex> lk(mu_);
    const Buffer *b = locate(req.tensor, req.offset, req.size, "get_tensor");
    if (!b) return false;
    try {
        out.resize(req.size);
    } catch (const std::exception &) {
        return false;
    }
    return req.size == 0 || backend_->download(b->dev, out.data(), reinterpret_cast<const void *>((uintptr_t)(req.tensor.data + req.offset)), req.size);
}

bool Server::copy_tensor(const CopyTensorReq &req) {
    std::lock_guard<std::mutex> lk(mu_);
    const uint64_t n = tensor_nbytes(req.src);
    if (n == 0 || n != tensor_nbytes(req.dst)) return false;
    const Buffer *s = locate(req.src, 0, n, "copy_tensor (source)");
    const Buffer *d = locate(req.dst, 0, n, "copy_tensor (destination)");
    if (!s || !d || s->dev != d->dev) return false;
    return backend_->copy(d->dev, reinterpret_cast<void *>((uintptr_t)req.dst.data), reinterpret_cast<const void *>((uintptr_t)req.src.data), n);
}

bool Server::set_tensor_gguf(const SetTensorGgufReq &req) {
    if (cfg_.gguf_path.empty()) return false;
    char name[MAX_NAME + 1];
    memcpy(name, req.tensor.name, MAX_NAME);
    name[MAX_NAME] = 0;
    mesh_tensor_info info;
    if (mesh_gguf_tensor(cfg_.gguf_path.c_str(), name, &info) != MESH_OK) {
        debug("set_tensor_gguf: '%s' not in %s (%s)", name, cfg_.gguf_path.c_str(), mesh_last_error());
        return false;
    }
    const uint64_t size = tensor_nbytes(req.tensor);
    if (size == 0 || size != info.nbytes || req.tensor.type != info.type) {
        log("set_tensor_gguf: '%s' is %llu bytes of type %u in the file, the request describes %llu bytes of type %u", name,
            (unsigned long long)info.nbytes, info.type, (unsigned long long)size, req.tensor.type);
        return false;
    }
    std::vector<uint8_t> data;
    try {
        data.resize(size);
    } catch (const std::exception &) {
        return false;
    }
    std::ifstream f(cfg_.gguf_path, std::ios::binary);
    if (!f.is_open()) return false;
    f.seekg((std::streamoff)info.file_offset);
    f.read(reinterpret_cast<char *>(data.data()), (std::streamsize)size);
    if (!f.good() || (uint64_t)f.gcount() != size) {
        log("set_tensor_gguf: short read of '%s'", name);
        return false;
    }
    std::lock_guard<std::mutex> lk(mu_);
    // the request's offset shifts the destination exactly as in the reference (ggml_backend_tensor_set(tensor, data, offset, size))
    const Buffer *b = locate(req.tensor, 0, size, "set_tensor_gguf");
    if (!b) return false;
    const uint64_t p1 = (uint64_t)(uintptr_t)b->base + b->size;
    if (req.offset > p1 - req.tensor.data || size > p1 - req.tensor.data - req.offset) return false;
    if (!backend_->upload(b->dev, reinterpret_cast<void *>((uintptr_t)(req.tensor.data + req.offset)), data.data(), size)) return false;
    log("loaded '%s' (%llu bytes) from local GGUF", name, (unsigned long long)size);
    return true;
}

bool Server::register_peer(const RegisterPeerReq &req) {
    const std::string endpoint(req.endpoint, strnlen(req.endpoint, sizeof req.endpoint));
    const size_t colon = endpoint.rfind(':');
    if (endpoint.empty() || colon == std::string::npos || colon == 0 || colon == endpoint.size() - 1) {
        log("register_peer: invalid endpoint '%s'", endpoint.c_str());
        return false;
    }
    std::lock_guard<std::mutex> lk(peers_mu_);
    peers_[req.peer_id] = Peer{endpoint, nullptr};      // (a re-registration drops the old link)
    debug("registered peer %u at %s", req.peer_id, endpoint.c_str());
    return true;
}

// The link to a registered peer, connected on first use.  The registry lock is held only to look the peer up and to publish
// a new link: connecting and the HELLO exchange happen outside it (the reference releases its lock before it talks to the
// peer, patches/0002:589-621), so one slow or dead peer does not stall pushes to the others.
std::shared_ptr<Server::PeerLink> Server::peer_link(uint32_t peer_id) {
    std::string endpoint;
    {
        std::lock_guard<std::mutex> lk(peers_mu_);
        auto it = peers_.find(peer_id);
        if (it == peers_.end()) {
            log("push: unknown peer %u", peer_id);
            return nullptr;
        }
        if (it->second.link) return it->second.link;
        endpoint = it->second.endpoint;
    }
    const size_t colon = endpoint.rfind(':');
    const std::string host = endpoint.substr(0, colon);
    const int port = atoi(endpoint.c_str() + colon + 1);
    std::shared_ptr<PeerLink> link(new PeerLink());
    link->conn = Conn::connect_to(host, port);
    if (!link->conn) {
        log("push: cannot connect to peer %u at %s", peer_id, endpoint.c_str());
        return nullptr;
    }
    const uint8_t cmd = CMD_HELLO;
    HelloReq hreq{};
    HelloRsp hrsp{};
    if (!link->conn->send_all(&cmd, 1) || !link->conn->send_msg(&hreq, sizeof hreq) || !link->conn->recv_msg(&hrsp, sizeof hrsp) || hrsp.major != PROTO_MAJOR) {
        log("push: peer %u at %s does not speak protocol %d.x", peer_id, endpoint.c_str(), PROTO_MAJOR);
        return nullptr;
    }
    std::lock_guard<std::mutex> lk(peers_mu_);
    auto it = peers_.find(peer_id);
    if (it == peers_.end() || it->second.endpoint != endpoint) return link;      // re-registered meanwhile: use this link once
    if (!it->second.link) it->second.link = link;                                // (another thread may have connected first: keep its link)
    return it->second.link;
}

bool Server::push_tensor_to_peer(const PushTensorToPeerReq &req) {
    // read the source range into host memory under the buffer lock, send it without the lock
    std::vector<uint8_t> payload;
    {
        std::lock_guard<std::mutex> lk(mu_);
        const Buffer *b = locate(req.src, req.offset, req.size, "push_tensor_to_peer");
        if (!b) return false;
        try {
            payload.resize(sizeof(Tensor) + sizeof(uint64_t) + req.size);
        } catch (const std::exception &) {
            return false;
        }
        memcpy(payload.data(), &req.dst, sizeof(Tensor));
        memcpy(payload.data() + sizeof(Tensor), &req.offset, sizeof(uint64_t));
        if (req.size && !backend_->download(b->dev, payload.data() + sizeof(Tensor) + sizeof(uint64_t),
                                            reinterpret_cast<const void *>((uintptr_t)(req.src.data + req.offset)), req.size))
            return false;
    }
    std::shared_ptr<PeerLink> link = peer_link(req.peer_id);
    if (!link) return false;
    const uint8_t cmd = CMD_PEER_TENSOR_DATA;
    uint8_t result = 0;
    bool sent;
    {
        std::lock_guard<std::mutex> io(link->io);          // this peer's connection only
        sent = link->conn->send_all(&cmd, 1) && link->conn->send_msg(payload.data(), payload.size()) && link->conn->recv_msg(&result, 1);
    }
    if (!sent) {
        log("push: lost the connection to peer %u", req.peer_id);
        std::lock_guard<std::mutex> lk(peers_mu_);
        auto it = peers_.find(req.peer_id);
        if (it != peers_.end() && it->second.link == link) it->second.link = nullptr;       // the next push connects again
        return false;
    }
    if (result != 1) log("push: peer %u rejected the tensor data", req.peer_id);
    return result == 1;
}

// ------------------------------------------------------------------------------------------------ graphs
// mu_ held.  The three tensors the run touches must lie inside live buffers of the graph's device.
bool Server::run_graph(const ParsedGraph &g) {
    if (g.device >= cfg_.devices.size()) {
        log("graph: device %u of %zu", g.device, cfg_.devices.size());
        return false;
    }
    const int dev = cfg_.devices[g.device];
    StagePlan plan;
    std::string why;
    if (!recognise_layer_range(g, &plan, &why)) {
        log("graph of %zu nodes refused: %s", g.nodes.size(), why.c_str());
        return false;
    }
    const Tensor *io[3] = {&plan.input, &plan.positions, &plan.output};
    const char *what[3] = {"graph (hidden-state input)", "graph (positions)", "graph (result)"};
    for (int i = 0; i < 3; ++i) {
        const Buffer *b = locate(*io[i], 0, tensor_nbytes(*io[i]), what[i]);
        if (!b) return false;
        if (b->dev != dev) {
            log("%s: tensor lives on another device than the graph's", what[i]);
            return false;
        }
    }
    // contiguous rows are what the stage reads and writes
    if (plan.input.nb[0] != 4 || plan.input.nb[1] != 4ull * plan.input.ne[0] || plan.output.nb[0] != 4 || plan.output.nb[1] != 4ull * plan.output.ne[0] ||
        plan.positions.nb[0] != 4) {
        log("graph refused: input, positions or result tensor is not contiguous");
        return false;
    }
    if (!graph_runner()->run(dev, cfg_.gguf_path, plan, &why)) {
        log("graph of layers [%d, %d), %d tokens failed: %s", plan.layer_begin, plan.layer_end, plan.n_tokens, why.c_str());
        return false;
    }
    debug("graph: layers [%d, %d), %d tokens%s", plan.layer_begin, plan.layer_end, plan.n_tokens, plan.logits ? ", logits" : "");
    return true;
}

bool Server::graph_compute(const std::vector<uint8_t> &input) {
    ParsedGraph g;
    std::string why;
    if (!parse_graph(input.data(), input.size(), &g, &why)) {
        log("graph_compute: malformed payload: %s", why.c_str());
        return false;
    }
    std::lock_guard<std::mutex> lk(mu_);
    if (!run_graph(g)) return false;
    stored_graphs_[g.device] = input;
    return true;
}

bool Server::graph_recompute(uint32_t device) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = stored_graphs_.find(device);
    if (it == stored_graphs_.end()) {
        log("graph_recompute: device %u has no stored graph", device);
        return false;
    }
    ParsedGraph g;
    std::string why;
    // parsed and checked again: buffers may have been freed since the graph ran
    if (!parse_graph(it->second.data(), it->second.size(), &g, &why)) return false;
    return run_graph(g);
}

// a serialized graph: 296 bytes per tensor; a 64-layer range has a few thousand
constexpr uint64_t GRAPH_PAYLOAD_LIMIT = (uint64_t)256 << 20;

void Server::serve_client(Conn &conn) {
    // a tensor payload cannot be larger than the largest live buffer it could land in
    auto payload_limit = [this]() {
        std::lock_guard<std::mutex> lk(mu_);
        uint64_t largest = 0;
        for (const auto &kv : buffers_) largest = std::max(largest, kv.second->size);
        return largest + sizeof(Tensor) + sizeof(uint64_t);
    };
    uint8_t cmd;
    if (!conn.recv_all(&cmd, 1)) return;
    if (cmd != CMD_HELLO) {
        log("expected HELLO as the first command, got %u", cmd);
        return;
    }
    {
        std::vector<uint8_t> hello;
        if (!conn.recv_msg(hello, sizeof(HelloReq)) || (hello.size() != 0 && hello.size() != sizeof(HelloReq))) return;
        HelloRsp rsp{};                 // no transport capabilities beyond plain TCP: conn_caps stay zero
        rsp.major = PROTO_MAJOR;
        rsp.minor = PROTO_MINOR;
        rsp.patch = PROTO_PATCH;
        if (!conn.send_msg(&rsp, sizeof rsp)) return;
    }
    const int n_dev = (int)cfg_.devices.size();
    for (;;) {
        if (!conn.recv_all(&cmd, 1)) return;
        if (cmd >= CMD_COUNT) {
            log("unknown command %u", cmd);
            return;
        }
        switch (cmd) {
            case CMD_HELLO:
                return;                 // only valid as the first command
            case CMD_DEVICE_COUNT: {
                if (!conn.recv_msg(nullptr, 0)) return;
                DeviceCountRsp rsp{(uint32_t)n_dev};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_GET_DEVICE_MEMORY: {
                GetDeviceMemoryReq req;
                if (!conn.recv_msg(&req, sizeof req) || req.device >= (uint32_t)n_dev) return;
                GetDeviceMemoryRsp rsp{};
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    if (!backend_->device_memory(cfg_.devices[req.device], &rsp.free_mem, &rsp.total_mem)) return;
                }
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_GET_ALIGNMENT: {
                GetAlignmentReq req;
                if (!conn.recv_msg(&req, sizeof req) || req.device >= (uint32_t)n_dev) return;
                GetAlignmentRsp rsp{backend_->alignment()};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_GET_MAX_SIZE: {
                GetMaxSizeReq req;
                if (!conn.recv_msg(&req, sizeof req) || req.device >= (uint32_t)n_dev) return;
                GetMaxSizeRsp rsp{backend_->max_size(cfg_.devices[req.device])};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_ALLOC_BUFFER: {
                AllocBufferReq req;
                if (!conn.recv_msg(&req, sizeof req) || req.device >= (uint32_t)n_dev) return;
                AllocBufferRsp rsp{0, 0};            // a failed allocation answers 0 / 0 and keeps the connection
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    const int dev = cfg_.devices[req.device];
                    void *base = backend_->alloc(dev, req.size);
                    if (base) {
                        std::unique_ptr<Buffer> b(new Buffer{base, req.size, dev});
                        rsp.remote_ptr = (uint64_t)(uintptr_t)b.get();
                        rsp.remote_size = req.size;
                        buffers_[rsp.remote_ptr] = std::move(b);
                    } else {
                        log("alloc_buffer: %llu bytes on device %u failed", (unsigned long long)req.size, req.device);
                    }
                }
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_BUFFER_GET_BASE: {
                BufferGetBaseReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                BufferGetBaseRsp rsp{0};
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    auto it = buffers_.find(req.remote_ptr);
                    if (it == buffers_.end()) {
                        log("buffer_get_base: buffer not found");
                        return;
                    }
                    rsp.base_ptr = (uint64_t)(uintptr_t)it->second->base;
                }
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_FREE_BUFFER: {
                FreeBufferReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    auto it = buffers_.find(req.remote_ptr);
                    if (it == buffers_.end()) {
                        log("free_buffer: buffer not found");
                        return;
                    }
                    backend_->release(it->second->dev, it->second->base);
                    buffers_.erase(it);
                }
                if (!conn.send_msg(nullptr, 0)) return;
                break;
            }
            case CMD_BUFFER_CLEAR: {
                BufferClearReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    auto it = buffers_.find(req.remote_ptr);
                    if (it == buffers_.end()) {
                        log("buffer_clear: buffer not found");
                        return;
                    }
                    if (!backend_->fill(it->second->dev, it->second->base, req.value, it->second->size)) return;
                }
                if (!conn.send_msg(nullptr, 0)) return;
                break;
            }
            case CMD_SET_TENSOR: {
                std::vector<uint8_t> input;
                if (!conn.recv_msg(input, payload_limit()) || !set_tensor(input)) return;
                break;                  // no reply
            }
            case CMD_SET_TENSOR_HASH: {
                SetTensorHashReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                SetTensorHashRsp rsp{0};             // no tensor cache in this build: the client sends the bytes
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_SET_TENSOR_GGUF: {
                SetTensorGgufReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                SetTensorGgufRsp rsp{(uint8_t)(set_tensor_gguf(req) ? 1 : 0)};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_INIT_TENSOR: {
                InitTensorReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                {
                    std::lock_guard<std::mutex> lk(mu_);
                    if (!locate(req.tensor, 0, 0, "init_tensor")) return;
                }
                if (!conn.send_msg(nullptr, 0)) return;     // plain HBM buffers need no per-tensor setup
                break;
            }
            case CMD_GET_ALLOC_SIZE: {
                GetAllocSizeReq req;
                if (!conn.recv_msg(&req, sizeof req) || req.device >= (uint32_t)n_dev) return;
                GetAllocSizeRsp rsp{tensor_nbytes(req.tensor)};
                if (rsp.alloc_size == 0) return;
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_GET_TENSOR: {
                GetTensorReq req;
                std::vector<uint8_t> out;
                if (!conn.recv_msg(&req, sizeof req) || !get_tensor(req, out)) return;
                if (!conn.send_msg(out.data(), out.size())) return;
                break;
            }
            case CMD_COPY_TENSOR: {
                CopyTensorReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                CopyTensorRsp rsp{(uint8_t)(copy_tensor(req) ? 1 : 0)};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_REGISTER_PEER: {
                RegisterPeerReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                RegisterPeerRsp rsp{(uint8_t)(register_peer(req) ? 1 : 0)};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_PUSH_TENSOR_TO_PEER: {
                PushTensorToPeerReq req;
                if (!conn.recv_msg(&req, sizeof req)) return;
                PushTensorToPeerRsp rsp{(uint8_t)(push_tensor_to_peer(req) ? 1 : 0)};
                if (!conn.send_msg(&rsp, sizeof rsp)) return;
                break;
            }
            case CMD_PEER_TENSOR_DATA: {
                std::vector<uint8_t> input;
                if (!conn.recv_msg(input, payload_limit())) return;
                const uint8_t result = set_tensor(input) ? 1 : 0;
                if (!conn.send_msg(&result, 1)) return;
                break;
            }
            case CMD_GRAPH_COMPUTE: {
                std::vector<uint8_t> input;
                if (!conn.recv_msg(input, GRAPH_PAYLOAD_LIMIT) || !graph_compute(input)) return;
                break;                  // no reply (patches/0002: the client does not wait for one)
            }
            case CMD_GRAPH_RECOMPUTE: {
                GraphRecomputeReq req;
                if (!conn.recv_msg(&req, sizeof req) || !graph_recompute(req.device)) return;
                break;                  // no reply
            }
            default:
                return;
        }
    }
}

// ------------------------------------------------------------------------------------------------ argv
static void print_devices(FILE *f, BufferBackend *backend) {
    fprintf(f, "available devices:\n");
    for (int i = 0; i < backend->device_count(); ++i) {
        uint64_t fr = 0, tot = 0;
        (void)backend->device_memory(i, &fr, &tot);
        fprintf(f, "  %s: %s (%llu MiB, %llu MiB free)\n", backend->device_name(i).c_str(), backend->device_description(i).c_str(),
                (unsigned long long)(tot >> 20), (unsigned long long)(fr >> 20));
    }
}

static void print_usage(const char *prog, const ServerConfig &cfg) {
    fprintf(stderr, "Usage: %s [options]\n\n", prog);
    fprintf(stderr, "options:\n");
    fprintf(stderr, "  -h, --help                       show this help message and exit\n");
    fprintf(stderr, "  -d, --device <dev1,dev2,...>     comma-separated list of devices\n");
    fprintf(stderr, "  -H, --host HOST                  host to bind to (default: %s)\n", cfg.host.c_str());
    fprintf(stderr, "  -p, --port PORT                  port to bind to (default: %d)\n", cfg.port);
    fprintf(stderr, "  -m, --gguf PATH                  local GGUF model file (enables zero-transfer tensor loading)\n");
    fprintf(stderr, "  -c, --cache                      accepted for compatibility; this build keeps no tensor cache\n");
    fprintf(stderr, "  -t, --threads N                  accepted for compatibility; no CPU backend here\n\n");
}

int parse_args(int argc, char **argv, BufferBackend *backend, ServerConfig *cfg) {
    const char *dbg = getenv("GGML_RPC_DEBUG");
    cfg->verbose = dbg && *dbg && strcmp(dbg, "0") != 0;
    for (int i = 1; i < argc; ++i) {
        const std::string arg = argv[i];
        auto value = [&](std::string *out) {
            if (++i >= argc) return false;
            *out = argv[i];
            return true;
        };
        std::string v;
        if (arg == "-h" || arg == "--help") {
            print_usage(argv[0], *cfg);
            return 1;
        } else if (arg == "-d" || arg == "--device") {
            if (!value(&v)) return 2;
            const int n = backend->device_count();
            size_t pos = 0;
            while (pos <= v.size()) {
                const size_t comma = v.find(',', pos);
                const std::string name = v.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
                int found = -1;
                for (int d = 0; d < n; ++d) {
                    const std::string dn = backend->device_name(d);       // "ROCm<i>"; "HIP<i>" is the same device
                    if (name == dn || name == "HIP" + std::to_string(d)) found = d;
                }
                if (found < 0) {
                    fprintf(stderr, "error: unknown device: %s\n", name.c_str());
                    print_devices(stderr, backend);
                    return 2;
                }
                cfg->devices.push_back(found);
                if (comma == std::string::npos) break;
                pos = comma + 1;
            }
        } else if (arg == "-H" || arg == "--host") {
            if (!value(&cfg->host)) return 2;
        } else if (arg == "-p" || arg == "--port") {
            if (!value(&v)) return 2;
            cfg->port = atoi(v.c_str());
            if (cfg->port <= 0 || cfg->port > 65535) {
                fprintf(stderr, "error: invalid port: %s\n", v.c_str());
                return 2;
            }
        } else if (arg == "-m" || arg == "--gguf") {
            if (!value(&cfg->gguf_path)) return 2;
        } else if (arg == "-c" || arg == "--cache") {
            // no tensor cache
        } else if (arg == "-t" || arg == "--threads") {
            if (!value(&v)) return 2;
        } else {
            fprintf(stderr, "error: unknown argument: %s\n", arg.c_str());
            print_usage(argv[0], *cfg);
            return 2;
        }
    }
    if (cfg->devices.empty())
        for (int d = 0; d < backend->device_count(); ++d) cfg->devices.push_back(d);
    if (cfg->devices.empty()) {
        fprintf(stderr, "error: no usable GPU\n");
        return 2;
    }
    return 0;
}

}  // namespace mesh_rpc
