"""A stand-in for mesh-llm's plugin host: listens on a unix socket, spawns the plugin with MESH_LLM_PLUGIN_ENDPOINT /
_TRANSPORT / _NAME as src/plugin/runtime.rs:186-188 does, and exchanges u32-length-prefixed protobuf Envelopes
(plugin/src/io.rs:166-184).  The message types are declared here from the field numbers of mesh-llm/proto/plugin.proto
and encoded / decoded by the protobuf runtime, so the plugin's hand-written wire code is checked against the real thing."""
import os
import socket
import struct
import subprocess

from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

F = descriptor_pb2.FieldDescriptorProto


def _build_messages():
    fd = descriptor_pb2.FileDescriptorProto(name="mesh_plugin_test.proto", package="meshllm.plugin.v1", syntax="proto3")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, number, ftype, label, tname in fields:
            f = m.field.add(name=fname, number=number, type=ftype, label=label)
            if tname:
                f.type_name = ".meshllm.plugin.v1." + tname
        return m

    O, R = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    msg("InitializeRequest", [("host_protocol_version", 1, F.TYPE_UINT32, O, None), ("host_version", 2, F.TYPE_STRING, O, None),
                              ("host_info_json", 3, F.TYPE_STRING, O, None), ("mesh_visibility", 4, F.TYPE_INT32, O, None)])
    msg("EndpointManifest", [("endpoint_id", 1, F.TYPE_STRING, O, None), ("kind", 2, F.TYPE_INT32, O, None), ("transport_kind", 3, F.TYPE_INT32, O, None),
                             ("protocol", 4, F.TYPE_STRING, O, None), ("address", 5, F.TYPE_STRING, O, None), ("args", 6, F.TYPE_STRING, R, None),
                             ("namespace", 7, F.TYPE_STRING, O, None), ("supports_streaming", 8, F.TYPE_BOOL, O, None), ("managed_by_plugin", 9, F.TYPE_BOOL, O, None)])
    msg("PluginManifest", [("endpoints", 7, F.TYPE_MESSAGE, R, "EndpointManifest"), ("capabilities", 8, F.TYPE_STRING, R, None)])
    msg("InitializeResponse", [("plugin_id", 1, F.TYPE_STRING, O, None), ("plugin_protocol_version", 2, F.TYPE_UINT32, O, None),
                               ("plugin_version", 3, F.TYPE_STRING, O, None), ("server_info_json", 4, F.TYPE_STRING, O, None),
                               ("capabilities", 5, F.TYPE_STRING, R, None), ("manifest", 6, F.TYPE_MESSAGE, O, "PluginManifest")])
    msg("HealthRequest", [])
    msg("HealthResponse", [("status", 1, F.TYPE_INT32, O, None), ("detail", 2, F.TYPE_STRING, O, None)])
    msg("ShutdownRequest", [("reason", 1, F.TYPE_STRING, O, None)])
    msg("ShutdownResponse", [])
    msg("RpcRequest", [("method", 1, F.TYPE_STRING, O, None), ("params_json", 2, F.TYPE_STRING, O, None)])
    msg("ErrorResponse", [("code", 1, F.TYPE_INT32, O, None), ("message", 2, F.TYPE_STRING, O, None), ("data_json", 3, F.TYPE_STRING, O, None)])
    env = msg("Envelope", [("protocol_version", 1, F.TYPE_UINT32, O, None), ("plugin_id", 2, F.TYPE_STRING, O, None), ("request_id", 3, F.TYPE_UINT64, O, None),
                           ("initialize_request", 10, F.TYPE_MESSAGE, O, "InitializeRequest"), ("initialize_response", 11, F.TYPE_MESSAGE, O, "InitializeResponse"),
                           ("health_request", 12, F.TYPE_MESSAGE, O, "HealthRequest"), ("health_response", 13, F.TYPE_MESSAGE, O, "HealthResponse"),
                           ("shutdown_request", 14, F.TYPE_MESSAGE, O, "ShutdownRequest"), ("shutdown_response", 15, F.TYPE_MESSAGE, O, "ShutdownResponse"),
                           ("rpc_request", 17, F.TYPE_MESSAGE, O, "RpcRequest"), ("error_response", 20, F.TYPE_MESSAGE, O, "ErrorResponse")])
    env.oneof_decl.add(name="payload")
    for f in env.field:
        if f.number >= 10:
            f.oneof_index = 0
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    cls = (lambda n: get(pool.FindMessageTypeByName("meshllm.plugin.v1." + n))) if get else \
          (lambda n: message_factory.MessageFactory(pool).GetPrototype(pool.FindMessageTypeByName("meshllm.plugin.v1." + n)))
    return {n: cls(n) for n in ("Envelope", "InitializeRequest", "InitializeResponse", "HealthRequest", "ShutdownRequest", "RpcRequest")}


PB = _build_messages()
PROTOCOL_VERSION = 2


class PluginHost:
    def __init__(self, binary, args, tmp_dir, name="stage-a"):
        self.name = name
        self.path = os.path.join(str(tmp_dir), "plugin.sock")
        if os.path.exists(self.path):
            os.unlink(self.path)
        self.listener = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
        self.listener.bind(self.path)
        self.listener.listen(1)
        self.listener.settimeout(120)
        env = dict(os.environ, MESH_LLM_PLUGIN_ENDPOINT=self.path, MESH_LLM_PLUGIN_TRANSPORT="unix", MESH_LLM_PLUGIN_NAME=name)
        self.proc = subprocess.Popen([binary, *args], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
        try:
            self.conn, _ = self.listener.accept()
        except socket.timeout:
            self.proc.kill()
            raise RuntimeError("plugin did not connect: " + self.proc.stdout.read().decode(errors="replace"))
        self.conn.settimeout(60)
        self.next_id = 1

    def _recv(self, n):
        out = b""
        while len(out) < n:
            c = self.conn.recv(n - len(out))
            if not c:
                raise EOFError()
            out += c
        return out

    def send_raw(self, body):
        self.conn.sendall(struct.pack("<I", len(body)) + body)

    def read_envelope(self):
        (n,) = struct.unpack("<I", self._recv(4))
        assert n <= 16 * 1024 * 1024
        env = PB["Envelope"]()
        env.ParseFromString(self._recv(n))
        return env

    def request(self, **payload):
        env = PB["Envelope"](protocol_version=PROTOCOL_VERSION, plugin_id=self.name, request_id=self.next_id)
        (field, value), = payload.items()
        getattr(env, field).CopyFrom(value)
        self.next_id += 1
        self.send_raw(env.SerializeToString())
        rsp = self.read_envelope()
        assert rsp.request_id == env.request_id and rsp.protocol_version == PROTOCOL_VERSION and rsp.plugin_id == self.name
        return rsp

    def initialize(self):
        return self.request(initialize_request=PB["InitializeRequest"](host_protocol_version=PROTOCOL_VERSION, host_version="0.65.0-test",
                                                                        host_info_json="{}", mesh_visibility=1))

    def close(self):
        try:
            self.conn.close()
        finally:
            self.listener.close()
            try:
                self.proc.wait(timeout=20)
            except subprocess.TimeoutExpired:
                self.proc.kill()
                self.proc.wait()
            out = self.proc.stdout.read().decode(errors="replace")
            self.proc.stdout.close()
        return out
