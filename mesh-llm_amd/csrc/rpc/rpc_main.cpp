// `rpc-server`: the executable mesh-llm spawns next to every serving node (mesh-llm/src/inference/launch.rs:887-1030,
// argv `-d DEV -p PORT [--gguf PATH]`; `-d <unknown>` lists the devices and fails, which is how the launcher probes them,
// launch.rs:768-782).

#include <csignal>
#include <cstdio>

#include "rpc_server.hpp"

int main(int argc, char **argv) {
    using namespace mesh_rpc;
    BufferBackend *backend = buffer_backend();
    ServerConfig cfg;
    const int rc = parse_args(argc, argv, backend, &cfg);
    if (rc != 0) return rc - 1;
    signal(SIGPIPE, SIG_IGN);
    Server server(backend, cfg);
    const int port = server.listen_on();
    if (port < 0) return 1;
    printf("Starting RPC server v%d.%d.%d\n", PROTO_MAJOR, PROTO_MINOR, PROTO_PATCH);
    printf("  endpoint       : %s:%d\n", cfg.host.c_str(), port);
    printf("  local GGUF     : %s\n", cfg.gguf_path.empty() ? "n/a" : cfg.gguf_path.c_str());
    printf("Devices:\n");
    for (size_t i = 0; i < cfg.devices.size(); ++i) {
        uint64_t fr = 0, tot = 0;
        (void)backend->device_memory(cfg.devices[i], &fr, &tot);
        printf("  %s: %s (%llu MiB, %llu MiB free)\n", backend->device_name(cfg.devices[i]).c_str(), backend->device_description(cfg.devices[i]).c_str(),
               (unsigned long long)(tot >> 20), (unsigned long long)(fr >> 20));
    }
    fflush(stdout);
    server.serve();
    return 0;
}
