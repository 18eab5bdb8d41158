// rpc-server-compatible front end of the stage library: the process mesh-llm starts per serving node
// (mesh-llm/src/inference/launch.rs:887-1030) and the peer of llama-server's RPC backend.  Buffer, tensor-transfer,
// local-GGUF load and server-to-server push commands are served; of graphs, the decoder sub-graph of a contiguous layer
// range is recognised and run as one stage decode call (rpc_graph.hpp), any other graph ends the connection with a logged
// reason, as a failing request does in the reference.
#pragma once

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "rpc_buffers.hpp"
#include "rpc_graph.hpp"
#include "rpc_wire.hpp"

namespace mesh_rpc {

// blocking byte stream over a connected TCP socket
class Conn {
  public:
    explicit Conn(int fd) : fd_(fd) {}
    ~Conn();
    Conn(const Conn &) = delete;
    Conn &operator=(const Conn &) = delete;
    bool send_all(const void *data, size_t size);
    bool recv_all(void *data, size_t size);
    // | size u64 | payload |
    bool send_msg(const void *data, uint64_t size);
    // fixed-size payload: the announced size must match
    bool recv_msg(void *data, uint64_t size);
    // variable payload, refused above `limit` bytes
    bool recv_msg(std::vector<uint8_t> &data, uint64_t limit);
    static std::unique_ptr<Conn> connect_to(const std::string &host, int port);

  private:
    int fd_;
};

struct ServerConfig {
    std::string host = "127.0.0.1";
    int port = 50052;
    std::vector<int> devices;           // backend device indices exposed as RPC devices 0..n-1
    std::string gguf_path;              // local model file for SET_TENSOR_GGUF, empty = none
    bool verbose = false;               // GGML_RPC_DEBUG=1
};

class Server {
  public:
    Server(BufferBackend *backend, ServerConfig cfg);
    ~Server();
    // binds and listens; returns the bound port (cfg.port, or the one the system chose for port 0 in tests), -1 on failure
    int listen_on();
    // accept loop: one thread per client; returns when stop() closes the listening socket
    void serve();
    // closes the listening socket, shuts the clients' sockets down and waits for their threads to leave (they touch the
    // buffers the destructor frees)
    void stop();
    // one client connection until it closes or sends something this build does not serve
    void serve_client(Conn &conn);

  private:
    struct Buffer {
        void *base;
        uint64_t size;
        int dev;                         // backend device index
    };
    // a connection to a peer server and the lock that keeps two pushes to that peer from interleaving on it
    struct PeerLink {
        std::unique_ptr<Conn> conn;
        std::mutex io;
    };
    struct Peer {
        std::string endpoint;
        std::shared_ptr<PeerLink> link;  // connected on first push
    };

    // the byte range [t.data + offset, + size) of a live buffer; nullptr with a logged reason otherwise
    const Buffer *locate(const Tensor &t, uint64_t offset, uint64_t size, const char *what);
    bool set_tensor(const std::vector<uint8_t> &input);
    bool get_tensor(const GetTensorReq &req, std::vector<uint8_t> &out);
    bool copy_tensor(const CopyTensorReq &req);
    bool set_tensor_gguf(const SetTensorGgufReq &req);
    bool register_peer(const RegisterPeerReq &req);
    bool push_tensor_to_peer(const PushTensorToPeerReq &req);
    std::shared_ptr<PeerLink> peer_link(uint32_t peer_id);
    // GRAPH_COMPUTE: parse, recognise, run, remember for GRAPH_RECOMPUTE (patches/0001:163-174: one stored graph per device)
    bool graph_compute(const std::vector<uint8_t> &input);
    bool graph_recompute(uint32_t device);
    bool run_graph(const ParsedGraph &g);
    void log(const char *fmt, ...) __attribute__((format(printf, 2, 3)));
    void debug(const char *fmt, ...) __attribute__((format(printf, 2, 3)));

    BufferBackend *backend_;
    ServerConfig cfg_;
    std::atomic<int> listen_fd_{-1};                         // read by the accept loop while stop() closes it
    std::mutex clients_mu_;
    std::condition_variable clients_cv_;
    std::unordered_set<int> client_fds_;                     // sockets of the running client threads
    std::mutex mu_;                                          // guards buffers_ and every backend call, like the reference's backend_mutex
    std::unordered_map<uint64_t, std::unique_ptr<Buffer>> buffers_;   // handle -> buffer
    std::unordered_map<uint32_t, std::vector<uint8_t>> stored_graphs_;  // RPC device -> payload of its last graph that ran (under mu_)
    std::mutex peers_mu_;                                    // guards the registry only, never held across network traffic
    std::unordered_map<uint32_t, Peer> peers_;
};

// rpc-server's argv (launch.rs:920-932: -d DEV -p PORT [--gguf PATH]; the reference's test harness adds -H HOST).
// Returns 0 to go on, or the process exit code + 1 when the process should end (help, bad arguments, device probe).
int parse_args(int argc, char **argv, BufferBackend *backend, ServerConfig *cfg);

}  // namespace mesh_rpc
