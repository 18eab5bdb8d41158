"""GPU parity of the boundary codec and the weight dequantizers, through the C ABI, against the CPU oracle
and the exact-rational golden vectors.  Bit-exact: these are integer/byte results."""
import numpy as np
import pytest

import oracle
from util import bits_equal_nan_aware, codec_input, mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _pack_dev(m, fmt, x_np, src_off=0, dst_off=0):
    """Pack through the device entry point; optional element/byte offsets force the unaligned path."""
    n = x_np.size
    src = torch.zeros(n + src_off, dtype=torch.float32, device="cuda")
    src[src_off:] = torch.from_numpy(x_np.reshape(-1)).cuda()
    nbytes = {m.Q8_0: n // 32 * 34, m.F16: n * 2, m.F32: n * 4}[fmt]
    dst = torch.zeros(nbytes + dst_off + 64, dtype=torch.uint8, device="cuda")
    m.act_pack_dev(fmt, src.data_ptr() + 4 * src_off, dst.data_ptr() + dst_off, n, _stream())
    torch.cuda.synchronize()
    out = dst.cpu().numpy()
    assert not out[:dst_off].any() and not out[dst_off + nbytes:].any(), "wrote outside the packed range"
    return out[dst_off:dst_off + nbytes]


def _unpack_dev(m, fmt, packed_np, n, src_off=0, dst_off=0):
    src = torch.zeros(packed_np.size + src_off, dtype=torch.uint8, device="cuda")
    src[src_off:] = torch.from_numpy(packed_np).cuda()
    dst = torch.full((n + dst_off + 16,), 7.0, dtype=torch.float32, device="cuda")
    m.act_unpack_dev(fmt, src.data_ptr() + src_off, dst.data_ptr() + 4 * dst_off, n, _stream())
    torch.cuda.synchronize()
    out = dst.cpu().numpy()
    assert np.all(out[:dst_off] == 7.0) and np.all(out[dst_off + n:] == 7.0), "wrote outside the output range"
    return out[dst_off:dst_off + n]


def test_q8_0_golden_vectors(golden):
    m = mesh()
    got = _pack_dev(m, m.Q8_0, golden["q8_0_x"])
    assert np.array_equal(got.reshape(-1, 34), golden["q8_0_blocks"])


def test_f16_golden_vectors(golden):
    m = mesh()
    x = golden["f16_x"]
    got = _pack_dev(m, m.F16, x).view(np.uint16)
    assert np.array_equal(got, golden["f16_bits"])


@pytest.mark.parametrize("T", [1, 16, 512, 4096])
def test_codec_config_bit_exact(T):
    m = mesh()
    x = codec_input(T)
    n = x.size
    # q8_0
    ref = oracle.quantize_q8_0(x.reshape(-1))
    got = _pack_dev(m, m.Q8_0, x)
    assert np.array_equal(got, ref)
    back = _unpack_dev(m, m.Q8_0, got, n)
    assert np.array_equal(back.view(np.uint32), oracle.dequantize(oracle.Q8_0, ref, n).view(np.uint32))
    # f16
    ref16 = oracle.fp32_to_fp16(x.reshape(-1))
    got16 = _pack_dev(m, m.F16, x).view(np.uint16)
    assert np.array_equal(got16, ref16)
    back16 = _unpack_dev(m, m.F16, got16.view(np.uint8), n)
    assert np.array_equal(back16.view(np.uint32), oracle.fp16_to_fp32(ref16).view(np.uint32))
    # f32 passthrough
    assert np.array_equal(_pack_dev(m, m.F32, x).view(np.float32), x.reshape(-1))
    # size-independent properties: every block's largest magnitude maps to +-127; error within half a step
    q = got.reshape(-1, 34)[:, 2:].view(np.int8)
    xb = x.reshape(-1, 32)
    am = np.argmax(np.abs(xb), axis=1)
    r = np.arange(xb.shape[0])
    assert np.array_equal(q[r, am], np.where(xb[r, am] > 0, 127, -127).astype(np.int8))
    step = np.abs(xb).max(axis=1, keepdims=True) / 127
    assert np.all(np.abs(back.reshape(-1, 32) - xb) <= step * 0.5001 + np.abs(xb) * 2.0**-10)


@pytest.mark.parametrize("nblk", [1, 2, 31, 255, 256, 257, 1000])
@pytest.mark.parametrize("src_off,dst_off", [(0, 0), (1, 0), (0, 2), (3, 6)])
def test_ragged_sizes_and_unaligned_pointers(nblk, src_off, dst_off):
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(nblk))
    x = (rng.standard_normal(nblk * 32) * 10.0 ** rng.integers(-3, 3, nblk * 32)).astype(np.float32)
    ref = oracle.quantize_q8_0(x)
    got = _pack_dev(m, m.Q8_0, x, src_off, dst_off)
    assert np.array_equal(got, ref)
    back = _unpack_dev(m, m.Q8_0, ref, x.size, dst_off, src_off)
    assert np.array_equal(back.view(np.uint32), oracle.dequantize(oracle.Q8_0, ref, x.size).view(np.uint32))
    # f16 with a count that is not a multiple of 8
    n16 = x.size - 3
    got16 = _pack_dev(m, m.F16, x[:n16], src_off, dst_off).view(np.uint16)
    assert np.array_equal(got16, oracle.fp32_to_fp16(x[:n16]))
    back16 = _unpack_dev(m, m.F16, got16.view(np.uint8), n16, dst_off, src_off)
    assert np.array_equal(back16.view(np.uint32), oracle.fp16_to_fp32(got16).view(np.uint32))


def test_f16_special_values():
    m = mesh()
    x = np.array([np.inf, -np.inf, np.nan, -np.nan, 65520.0, 65519.996, 2.0**-24, 2.0**-25, -(2.0**-25) * 1.0001,
                  1e-10, -0.0, 0.0, 70000.0, 5.9604645e-08, 6.1035156e-05, 6.0975552e-05], dtype=np.float32)
    got = _pack_dev(m, m.F16, x).view(np.uint16)
    assert np.array_equal(got, oracle.fp32_to_fp16(x))
    # all 65536 halves decode exactly
    h = np.arange(65536, dtype=np.uint16)
    back = _unpack_dev(m, m.F16, h.view(np.uint8), h.size)
    assert bits_equal_nan_aware(back, h.view(np.float16).astype(np.float32))


def test_host_pointer_entry_points():
    m = mesh()
    x = codec_input(16)
    ref = oracle.quantize_q8_0(x.reshape(-1))
    got = m.act_pack(m.Q8_0, x)
    assert np.array_equal(got, ref)
    assert np.array_equal(m.act_unpack(m.Q8_0, got, x.size), oracle.dequantize(oracle.Q8_0, ref, x.size))
    assert np.array_equal(m.act_pack(m.F16, x).view(np.uint16), oracle.fp32_to_fp16(x.reshape(-1)))
    assert np.array_equal(m.act_unpack(m.F32, m.act_pack(m.F32, x), x.size), x.reshape(-1))


def test_all_zero_and_constant_blocks():
    m = mesh()
    x = np.zeros(64, np.float32)
    x[32:] = -3.25
    got = _pack_dev(m, m.Q8_0, x).reshape(2, 34)
    assert not got[0].any()
    assert np.all(got[1, 2:].view(np.int8) == -127)
    assert np.array_equal(got.reshape(-1), oracle.quantize_q8_0(x))


@pytest.mark.parametrize("name,type_,be,bb", [("q4_K", 12, 256, 144), ("q6_K", 14, 256, 210), ("q5_0", 6, 32, 22), ("q8_0", 8, 32, 34)])
def test_weight_dequant_bit_exact(golden, name, type_, be, bb):
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(type_))
    blocks = [rng.integers(0, 256, 2048 * bb, dtype=np.uint8)]
    if name + "_blocks" in golden:
        blocks.append(golden[name + "_blocks"].reshape(-1))
    for data in blocks:
        n = data.size // bb * be
        src = torch.from_numpy(data).cuda()
        dst = torch.empty(n, dtype=torch.float32, device="cuda")
        m.dequantize_dev(type_, src.data_ptr(), dst.data_ptr(), n, _stream())
        torch.cuda.synchronize()
        assert bits_equal_nan_aware(dst.cpu().numpy(), oracle.dequantize(type_, data, n))
    if name + "_y" in golden:
        assert np.array_equal(dst.cpu().numpy().view(np.uint32), golden[name + "_y"].reshape(-1).view(np.uint32))


def test_device_entry_points_reject_bad_arguments():
    m = mesh()
    buf = torch.zeros(1024, dtype=torch.float32, device="cuda")
    with pytest.raises(m.MeshError) as e:
        m.act_pack_dev(m.Q8_0, buf.data_ptr(), buf.data_ptr(), 33, _stream())
    assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError):
        m.act_pack_dev(m.Q8_0, 0, buf.data_ptr(), 32, _stream())
    with pytest.raises(m.MeshError):
        m.dequantize_dev(m.Q4_K, buf.data_ptr(), buf.data_ptr(), 100, _stream())
    m.device_select("ROCm0")
    m.device_select("HIP0")
    assert m.device_count() >= 1


def test_hbm_read_probe_reports_plausible_bandwidth():
    """The streaming-read yardstick (protocol of mesh-llm/benchmarks/membench-fingerprint.hip): 5 timed passes over
    256 MiB, each between 1 and 10 TB/s on an MI355X."""
    m = mesh()
    g = m.hbm_read_probe(256 << 20, 2, 5)
    assert len(g) == 5 and all(1000.0 < v < 10000.0 for v in g), g
