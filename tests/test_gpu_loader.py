"""GGUF file -> device: the loader of the host layer drives the HIP kernels from real container files."""
import base64
import json
import os

import numpy as np
import pytest

import oracle
from gguf_writer import write_gguf
from nntrain_amd import (BLOCK_BYTES, BLOCK_ELEMS, GGML_BF16, GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0,
                         GgufReader, HipExecutionLane, HipGgufLoader, HipQuantizedMatrix, NotSupportedError, synth)
from nntrain_amd.native import NnHipError

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("staged", [True, False])
def test_loader_reference_file_drives_the_kernels(lane, golden_dir, staged):
    """The gguf-py written fixture, loaded through the loader (file -> pinned staging -> device inside the library, or
    read here and uploaded piece by piece): decode bit-exact, linear within the reference's bound
    (QwenGgufIndependentReferenceTests.cs:18-43,76-97), dense tensors widened exactly, nothing left on the host."""
    expected = json.loads((golden_dir / "qwen_gguf_expected.json").read_text())
    K, N = expected["inputWidth"], expected["outputWidth"]
    x_all = np.frombuffer(base64.b64decode(expected["inputFloat32Base64"]), "<f4").reshape(expected["inputRows"], K)
    with GgufReader(str(golden_dir / "qwen_gguf_reference.gguf")) as reader:
        before = lane.counters()
        loader = HipGgufLoader(lane, reader, chunk_bytes=1000, staged=staged)          # pieces that cut through blocks
        matrices, dense = loader.load_all()
        after = lane.counters()
        assert sorted(matrices) == sorted(t["name"] for t in expected["tensors"] if t["type"] in (GGML_Q4_K, GGML_Q6_K))
        assert sorted(dense) == ["f16_edges", "f32_edges"]
        quant_bytes = sum(t["payloadBytes"] for t in expected["tensors"] if t["name"] in matrices)
        assert loader.quantized_bytes == quant_bytes
        assert after["h2d_bytes"] - before["h2d_bytes"] == quant_bytes + loader.dense_bytes
        xb = lane.upload_raw(x_all)
        for t in expected["tensors"]:
            want = np.frombuffer(base64.b64decode(t["decodedFloat32Base64"]), "<f4")
            if t["name"] in dense:
                assert np.array_equal(_bits(lane.read(dense[t["name"]], count=want.size)), _bits(want))
                continue
            mat = matrices[t["name"]]
            assert (mat.ggml_type, mat.input_width, mat.output_width) == (t["type"], K, N)
            assert mat.storage_bytes == t["payloadBytes"]
            assert np.array_equal(_bits(lane.read(mat.dequantize(lane))), _bits(want))
            bias = np.frombuffer(base64.b64decode(t["biasFloat32Base64"]), "<f4")
            ref = np.frombuffer(base64.b64decode(t["linearFloat64Base64"]), "<f8").reshape(-1, N)
            bb = lane.upload_raw(bias)
            y = lane.read(mat.forward(lane, xb, bb, ref.shape[0])).reshape(-1, N)
            assert np.max(np.abs(y - ref)) <= np.max(np.abs(ref)) * 5e-6 + 1e-9
            bb.dispose()
        for m in matrices.values():
            m.dispose()


def test_loader_all_block_formats_and_dense_kinds(lane, tmp_path):
    """A file with every block format of the path plus F32/F16/BF16 tensors: what the loader puts on the device is
    byte-identical to a direct upload (same kernel results bit for bit), whatever the piece size."""
    rng = np.random.default_rng(77)
    specs = [(GGML_Q8_0, 160, 9), (GGML_Q4_K, 512, 5), (GGML_Q5_K, 256, 3), (GGML_Q6_K, 768, 4), (GGML_IQ3_S, 512, 6),
             (GGML_IQ2_S, 256, 7), (GGML_BF16, 192, 5)]
    tensors, payloads = [], {}
    for typ, in_w, out_w in specs:
        p = synth.matrix(typ, out_w, in_w, 900 + typ)
        payloads[f"m{typ}.weight"] = (typ, in_w, out_w, p)
        tensors.append((f"m{typ}.weight", (in_w, out_w), typ, p.tobytes()))
    f32 = rng.standard_normal(33).astype(np.float32)
    f16 = rng.standard_normal(20).astype(np.float16)
    bf16 = synth.to_bf16_bits(rng.standard_normal(12).astype(np.float32))
    tensors += [("n32", (33,), 0, f32.tobytes()), ("n16", (4, 5), 1, f16.tobytes()), ("nb", (12,), 30, bf16.tobytes())]
    path = write_gguf(tmp_path / "all.gguf", tensors)
    with GgufReader(path) as reader:
        for chunk, staged in ((97, False), (1 << 20, False), (1 << 20, True)):
            matrices, dense = HipGgufLoader(lane, reader, chunk_bytes=chunk, staged=staged).load_all()
            assert set(matrices) == set(payloads) and set(dense) == {"n32", "n16", "nb"}
            assert np.array_equal(_bits(lane.read(dense["n32"], count=33)), _bits(f32))
            assert np.array_equal(_bits(lane.read(dense["n16"], count=20)), _bits(f16.astype(np.float32)))
            assert np.array_equal(lane.read(dense["nb"], np.uint32, 12), bf16.astype(np.uint32) << 16)
            for name, (typ, in_w, out_w, p) in payloads.items():
                mat = matrices[name]
                x = synth.activations(2, in_w, 5)
                xb = lane.upload_raw(x)
                direct = HipQuantizedMatrix(p, typ, out_w, in_w)
                y_loaded = lane.read(mat.forward(lane, xb, None, 2))
                y_direct = lane.read(direct.forward(lane, xb, None, 2))
                assert np.array_equal(_bits(y_loaded), _bits(y_direct)), name
                ref, _ = oracle.linear_f64(typ, p, x, None, 2, in_w, out_w)
                assert oracle.rel_l2(y_loaded.reshape(2, out_w), ref) <= 1e-5
                assert np.array_equal(_bits(lane.read(mat.dequantize(lane, row=out_w - 1))),
                                      _bits(oracle.dequantize(typ, p)[-in_w:]))
                with pytest.raises(ValueError, match="host payload was dropped|bound"):
                    other = HipExecutionLane(0)
                    try:
                        mat.device_payload(other)
                    finally:
                        other.dispose()
                direct.dispose()
                xb.dispose()
            for m in matrices.values():
                m.dispose()
            for b in dense.values():
                b.dispose()


def test_loader_rejects_what_it_cannot_hold(lane, tmp_path):
    path = write_gguf(tmp_path / "bad.gguf", [("ok.weight", (256, 2), GGML_Q4_K, bytes(288)),
                                               ("odd", (256,), GGML_Q4_K, bytes(144)),          # 1-D quantized tensor
                                               ("i8", (8,), 24, bytes(8))])                      # GGML_TYPE_I8
    with GgufReader(path) as reader:
        loader = HipGgufLoader(lane, reader)
        before = lane.counters()["allocated_bytes"]
        with pytest.raises(NotSupportedError, match="F32/F16/BF16"):
            loader.load_all()
        assert lane.counters()["allocated_bytes"] == before          # what was uploaded before the failure is released
        m = loader.load_matrix("ok.weight")
        assert (m.input_width, m.output_width) == (256, 2)
        m.dispose()
        with pytest.raises(KeyError):
            loader.load_matrix("missing.weight")
        with pytest.raises(ValueError):
            HipGgufLoader(lane, reader, chunk_bytes=0)


def test_upload_from_file_moves_the_exact_bytes(lane, tmp_path):
    """nnhip_upload_from_file: a range of several staging buffers (16 MiB each) plus a ragged end, from a file offset
    and to a device offset that are not multiples of anything, lands byte for byte; the bytes around it stay; the
    descriptor's own position is not moved; a second, shorter call reuses the buffers."""
    rng = np.random.default_rng(5)
    data = rng.integers(0, 256, size=(40 << 20) + 12345, dtype=np.uint8)
    path = tmp_path / "blob.bin"
    path.write_bytes(data.tobytes())
    fd = os.open(path, os.O_RDONLY)
    try:
        buf = lane.allocate_bytes((data.size + 4096) // 4 * 4)
        lane.fill_u32(buf, 0xA5A5A5A5, buf.nbytes // 4)
        before = lane.counters()["h2d_bytes"]
        file_off, dev_off, n = 777, 1031, data.size - 777 - 99
        os.lseek(fd, 4242, os.SEEK_SET)
        lane.write_from_file(buf, fd, file_off, n, offset=dev_off)
        assert os.lseek(fd, 0, os.SEEK_CUR) == 4242
        assert lane.counters()["h2d_bytes"] - before == n
        got = lane.read(buf, np.uint8)
        assert np.array_equal(got[dev_off:dev_off + n], data[file_off:file_off + n])
        assert np.all(got[:dev_off] == 0xA5) and np.all(got[dev_off + n:] == 0xA5)
        # a short range right after a long one (the staging buffers still hold the long one's tail)
        lane.write_from_file(buf, fd, 5, 1000, offset=0)
        got = lane.read(buf, np.uint8, 2000)
        assert np.array_equal(got[:1000], data[5:1005]) and np.all(got[1000:dev_off] == 0xA5)
        lane.write_from_file(buf, fd, 0, 0)                                     # nothing to do
        # a range that runs past the end of the file: reported, and what arrived is counted
        before = lane.counters()["h2d_bytes"]
        with pytest.raises(NnHipError, match="file ends 50 bytes before"):
            lane.write_from_file(buf, fd, data.size - 100, 150)
        assert lane.counters()["h2d_bytes"] - before == 0
        with pytest.raises(ValueError):
            lane.write_from_file(buf, fd, 0, buf.nbytes + 1)
        with pytest.raises(NnHipError, match="descriptor"):
            lane.write_from_file(buf, -1, 0, 16)
        closed = os.open(path, os.O_RDONLY)
        os.close(closed)
        with pytest.raises(NnHipError, match="reading the file failed"):
            lane.write_from_file(buf, closed, 0, 16)
        buf.dispose()
    finally:
        os.close(fd)
