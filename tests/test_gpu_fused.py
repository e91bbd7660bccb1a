"""GPU parity of the fused decode mat-vec (activation preparation + mat-vec + residual add in one launch).

Bar: bit-identical to the unfused sequence of this library's own entry points (nnhip_add_rms_norm / nnhip_rms_norm /
nnhip_silu_multiply, nnhip_quant_matvec, nnhip_add_in_place), each of which is checked against the oracle elsewhere;
and, end to end, within the mat-vec bar (relative L2 <= 1e-5) of the float64 oracle fed the oracle's own FP32
preparation.
"""
import numpy as np
import pytest

import oracle
from nntrain_amd import (GGML_BF16, GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, HipExecutionLane,
                         HipQuantizedMatrix, NnHipError, qwen35_gpu, synth)
from nntrain_amd.native import POST_SILU_PAIR
from nntrain_amd.quantized_matrix import PRE_NONE, PRE_RMS_NORM, PRE_SILU_MULTIPLY

pytestmark = pytest.mark.gpu

TYPES = [GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ3_S, GGML_IQ2_S, GGML_BF16]
SHAPES = [(256, 8), (1024, 67), (5120, 131)]           # (in_w, out_w); 17408 is covered separately (staging loop)
EPS = 1e-6


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _matrix(typ, out_w, in_w, seed):
    return HipQuantizedMatrix(synth.matrix(typ, out_w, in_w, seed), typ, out_w, in_w)


def _vectors(in_w, out_w, seed):
    rng = np.random.default_rng(seed)
    f = lambda n, s=1.0: (rng.standard_normal(n) * s).astype(np.float32)     # noqa: E731
    return dict(hidden=f(in_w, 3), residual=f(in_w), gamma=rng.uniform(-2, 2, in_w).astype(np.float32), gate=f(in_w, 4),
                up=f(in_w), bias=f(out_w, 0.1), stream=f(out_w, 2))


@pytest.mark.parametrize("typ", TYPES)
@pytest.mark.parametrize("in_w,out_w", SHAPES)
def test_rms_norm_projection_equals_the_unfused_sequence_bitwise(lane, typ, in_w, out_w):
    v = _vectors(in_w, out_w, in_w + typ)
    m = _matrix(typ, out_w, in_w, 3)
    up = lambda a: lane.upload_raw(a)                                           # noqa: E731
    for with_residual in (True, False):
        hid_a, hid_b, res, gam, bias = up(v["hidden"]), up(v["hidden"]), up(v["residual"]), up(v["gamma"]), up(v["bias"])
        # unfused: (hidden += residual) -> RMSNorm -> mat-vec
        if with_residual:
            norm = qwen35_gpu.add_residual_and_rms_norm(lane, hid_a, res, gam, in_w, EPS)
        else:
            norm = qwen35_gpu.rms_norm(lane, hid_a, gam, 1, in_w, EPS)
        y_ref = m.forward(lane, norm, bias)
        # fused
        x_out, sum_out = lane.allocate(in_w), lane.allocate(in_w)
        y = m.forward_fused(lane, hid_b, pre_op=PRE_RMS_NORM, x2=res if with_residual else None, norm_weight=gam,
                            epsilon=EPS, x_out=x_out, sum_out=sum_out if with_residual else None, bias=bias)
        assert np.array_equal(_bits(lane.read(x_out, count=in_w)), _bits(lane.read(norm, count=in_w)))
        if with_residual:
            assert np.array_equal(_bits(lane.read(sum_out, count=in_w)), _bits(lane.read(hid_a, count=in_w)))
        assert np.array_equal(_bits(lane.read(hid_b, count=in_w)), _bits(v["hidden"]))      # the fused form writes elsewhere
        assert np.array_equal(_bits(lane.read(y, count=out_w)), _bits(lane.read(y_ref, count=out_w)))
        for b in (hid_a, hid_b, res, gam, bias, norm, y_ref, x_out, sum_out, y):
            b.dispose()
    m.dispose()


@pytest.mark.parametrize("typ", TYPES)
@pytest.mark.parametrize("in_w,out_w", SHAPES + [(17408, 33)])
def test_silu_down_projection_and_residual_add_equal_the_unfused_sequence_bitwise(lane, typ, in_w, out_w):
    v = _vectors(in_w, out_w, in_w + 7 * typ)
    m = _matrix(typ, out_w, in_w, 4)
    gate, upv, stream_a, stream_b = (lane.upload_raw(v[k]) for k in ("gate", "up", "stream", "stream"))
    act = qwen35_gpu.silu_multiply(lane, gate, upv, in_w)
    down = m.forward(lane, act, None)
    qwen35_gpu.add_in_place(lane, stream_a, down, out_w)
    x_out = lane.allocate(in_w)
    y = m.forward_fused(lane, gate, pre_op=PRE_SILU_MULTIPLY, x2=upv, x_out=x_out, addend=stream_b, out=stream_b)
    assert y is stream_b
    assert np.array_equal(_bits(lane.read(x_out, count=in_w)), _bits(lane.read(act, count=in_w)))
    assert np.array_equal(_bits(lane.read(stream_b, count=out_w)), _bits(lane.read(stream_a, count=out_w)))
    for b in (gate, upv, stream_a, stream_b, act, down, x_out):
        b.dispose()
    m.dispose()


@pytest.mark.parametrize("typ", TYPES)
@pytest.mark.parametrize("in_w,half", [(256, 5), (1024, 67), (5120, 300), (5376, 1031)])
def test_stacked_gate_up_with_silu_pair_equals_the_unfused_sequence_bitwise(lane, typ, in_w, half):
    """NNHIP_POST_SILU_PAIR: y[o] = SiLU(z[o]) * z[half + o], against projection -> nnhip_silu_multiply of the two halves;
    with and without the RMSNorm in front, with a bias, odd halves and halves that do not fill the last row step."""
    if typ == GGML_Q8_0 and (in_w // 32) % 2:
        pytest.skip("rows of an odd number of Q8_0 blocks are not covered by the fused entry")
    out_w = 2 * half
    v = _vectors(in_w, out_w, in_w + 3 * typ)
    m = _matrix(typ, out_w, in_w, 6)
    x, gam, bias = lane.upload_raw(v["hidden"]), lane.upload_raw(v["gamma"]), lane.upload_raw(v["bias"])
    for pre in (PRE_NONE, PRE_RMS_NORM):
        vec = x if pre == PRE_NONE else qwen35_gpu.rms_norm(lane, x, gam, 1, in_w, EPS)
        z = m.forward(lane, vec, bias)
        ref = qwen35_gpu.silu_multiply(lane, z.view(0, 4 * half), z.view(4 * half, 4 * half), half)
        y = lane.allocate(half + 3)
        lane.fill_u32(y, 0x7FC00000, half + 3)
        m.forward_fused(lane, x, pre_op=pre, norm_weight=gam if pre else None, epsilon=EPS if pre else 0.0, bias=bias,
                        out=y, post_op=POST_SILU_PAIR)
        got = lane.read(y, count=half + 3)
        assert np.array_equal(_bits(got[:half]), _bits(lane.read(ref, count=half))), (typ, in_w, half, pre)
        assert np.all(np.isnan(got[half:]))                       # nothing is written past the half
        for b in (z, ref, y) + ((vec,) if pre else ()):
            b.dispose()
    for b in (x, gam, bias):
        b.dispose()
    m.dispose()


@pytest.mark.parametrize("typ", [GGML_Q8_0, GGML_Q4_K, GGML_Q6_K, GGML_IQ3_S, GGML_BF16])
@pytest.mark.parametrize("heads,kv,width,out_w", [(8, 2, 64, 37), (32, 16, 128, 300), (6, 6, 128, 9)])
def test_head_gather_equals_first_token_attention_then_projection_bitwise(lane, typ, heads, kv, width, out_w):
    """x_head_width / x_head_group: the o projection reads the value heads itself; with the residual stream as addend."""
    in_w = heads * width
    if typ == GGML_Q8_0 and (in_w // 32) % 2:
        pytest.skip("rows of an odd number of Q8_0 blocks are not covered by the fused entry")
    if in_w % 256:
        pytest.skip("in_w is not a whole number of blocks")
    rng = np.random.default_rng(heads + kv)
    values = rng.standard_normal(kv * width).astype(np.float32)
    stream = rng.standard_normal(out_w).astype(np.float32)
    m = _matrix(typ, out_w, in_w, 8)
    vb, sa, sb = lane.upload_raw(values), lane.upload_raw(stream), lane.upload_raw(stream)
    ctx = qwen35_gpu.first_token_attention(lane, vb, heads, kv, width)
    attn = m.forward(lane, ctx, None)
    qwen35_gpu.add_in_place(lane, sa, attn, out_w)
    out = m.forward_fused(lane, vb, addend=sb, out=sb, x_head_width=width, x_head_group=heads // kv)
    assert out is sb
    assert np.array_equal(_bits(lane.read(sb, count=out_w)), _bits(lane.read(sa, count=out_w)))
    for b in (vb, sa, sb, ctx, attn):
        b.dispose()
    m.dispose()


def test_new_descriptor_fields_are_checked(lane):
    m = _matrix(GGML_Q4_K, 64, 1024, 2)
    x, y, stream = lane.allocate(1024), lane.allocate(64), lane.allocate(64)
    bad = [dict(post_op=2), dict(post_op=POST_SILU_PAIR, addend=stream), dict(x_head_width=128, x_head_group=0),
           dict(x_head_width=130, x_head_group=1), dict(x_head_width=128, x_head_group=3),
           dict(x_head_width=128, x_head_group=2, pre_op=PRE_RMS_NORM, norm_weight=x, epsilon=EPS),
           dict(post_op=POST_SILU_PAIR, pre_op=PRE_SILU_MULTIPLY, x2=x)]
    for kw in bad:
        with pytest.raises(NnHipError) as info:
            m.forward_fused(lane, x, out=y, **kw)
        assert info.value.status == 1, kw
    odd = _matrix(GGML_Q4_K, 65, 1024, 2)
    with pytest.raises(NnHipError):
        odd.forward_fused(lane, x, out=y, post_op=POST_SILU_PAIR)
    for b in (x, y, stream):
        b.dispose()
    m.dispose()
    odd.dispose()


@pytest.mark.parametrize("typ", [GGML_Q8_0, GGML_Q4_K, GGML_IQ2_S])
def test_plain_with_addend_and_without_outputs(lane, typ):
    in_w, out_w = 2048, 517
    v = _vectors(in_w, out_w, 11)
    m = _matrix(typ, out_w, in_w, 5)
    x, bias, stream = lane.upload_raw(v["gate"]), lane.upload_raw(v["bias"]), lane.upload_raw(v["stream"])
    y_ref = lane.read(m.forward(lane, x, bias), count=out_w)
    y = m.forward_fused(lane, x, pre_op=PRE_NONE, bias=bias, addend=stream)
    assert np.array_equal(_bits(lane.read(y, count=out_w)), _bits(v["stream"] + y_ref))
    # pre-ops without the optional outputs
    gam = lane.upload_raw(v["gamma"][:in_w])
    a = m.forward_fused(lane, x, pre_op=PRE_RMS_NORM, norm_weight=gam, epsilon=EPS)
    norm = qwen35_gpu.rms_norm(lane, x, gam, 1, in_w, EPS)
    assert np.array_equal(_bits(lane.read(a, count=out_w)), _bits(lane.read(m.forward(lane, norm, None), count=out_w)))
    m.dispose()


@pytest.mark.parametrize("typ", [GGML_Q8_0, GGML_Q4_K, GGML_Q6_K])
def test_feed_forward_half_of_a_layer_against_the_float64_oracle(lane, typ):
    # hidden += attention; n = RMSNorm(hidden); hidden += W_down (SiLU(W_gate n) * (W_up n))   (Qwen35QuantizedModel.cs:486-498)
    width, ffn = 1024, 2816 if typ == GGML_Q8_0 else 2816 - 2816 % 256
    rng = np.random.default_rng(21)
    hidden = (rng.standard_normal(width) * 2).astype(np.float32)
    attn = rng.standard_normal(width).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, width).astype(np.float32)
    raw = {k: synth.matrix(typ, o, i, s) for k, (o, i, s) in dict(gate=(ffn, width, 1), up=(ffn, width, 2), down=(width, ffn, 3)).items()}
    mats = {k: HipQuantizedMatrix(raw[k], typ, *(dict(gate=(ffn, width), up=(ffn, width), down=(width, ffn))[k])) for k in raw}
    hb, ab, gb = lane.upload_raw(hidden), lane.upload_raw(attn), lane.upload_raw(gamma)
    stream, normed = lane.allocate(width), lane.allocate(width)
    launches = lane.counters()["kernel_launches"]
    g = mats["gate"].forward_fused(lane, hb, pre_op=PRE_RMS_NORM, x2=ab, norm_weight=gb, epsilon=EPS, x_out=normed, sum_out=stream)
    u = mats["up"].forward(lane, normed, None)
    mats["down"].forward_fused(lane, g, pre_op=PRE_SILU_MULTIPLY, x2=u, addend=stream, out=stream)
    assert lane.counters()["kernel_launches"] - launches == 3              # the reference issues six
    got = lane.read(stream, count=width)
    # oracle: FP32 row operations, float64 mat-vecs
    summed, n = oracle.add_rms_norm(hidden, attn, gamma, 1, width, EPS)
    g64, _ = oracle.linear_f64(typ, raw["gate"], n.ravel(), None, 1, width, ffn)
    u64, _ = oracle.linear_f64(typ, raw["up"], n.ravel(), None, 1, width, ffn)
    act = oracle.silu_multiply(g64.astype(np.float32).ravel(), u64.astype(np.float32).ravel())
    d64, _ = oracle.linear_f64(typ, raw["down"], act, None, 1, ffn, width)
    want = summed.astype(np.float64) + d64.ravel()
    assert oracle.rel_l2(got, want) <= 1e-5
    for m in mats.values():
        m.dispose()


def test_argument_checks(lane):
    m = _matrix(GGML_Q4_K, 8, 256, 1)
    x, small = lane.allocate(256), lane.allocate(8)
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=PRE_RMS_NORM)                              # no norm weight
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=PRE_RMS_NORM, norm_weight=x, epsilon=-1.0)
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=PRE_SILU_MULTIPLY)                         # no up vector
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=PRE_SILU_MULTIPLY, x2=x, x_out=x)          # output over an input
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=PRE_NONE, x2=x)
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, pre_op=7)
    with pytest.raises(ValueError):
        m.forward_fused(lane, x, pre_op=PRE_SILU_MULTIPLY, x2=small)
    odd = HipQuantizedMatrix(synth.matrix(GGML_Q8_0, 4, 96, 1), GGML_Q8_0, 4, 96)
    with pytest.raises(NnHipError):
        odd.forward_fused(lane, x, pre_op=PRE_NONE)                                # three Q8_0 blocks per row
    m.dispose()
    odd.dispose()


@pytest.mark.parametrize("typ", [GGML_Q8_0, GGML_Q4_K, GGML_Q6_K, GGML_IQ2_S])
def test_stacked_gate_and_up_make_a_two_launch_feed_forward(lane, typ):
    width, ffn = 1024, 2816 if typ == GGML_Q8_0 else 2560
    rng = np.random.default_rng(31)
    hidden = (rng.standard_normal(width) * 2).astype(np.float32)
    attn = rng.standard_normal(width).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, width).astype(np.float32)
    gate, up, down = _matrix(typ, ffn, width, 1), _matrix(typ, ffn, width, 2), _matrix(typ, width, ffn, 3)
    hb, ab, gb = lane.upload_raw(hidden), lane.upload_raw(attn), lane.upload_raw(gamma)
    # three launches, separate gate and up
    stream, normed = lane.allocate(width), lane.allocate(width)
    g = gate.forward_fused(lane, hb, pre_op=PRE_RMS_NORM, x2=ab, norm_weight=gb, epsilon=EPS, x_out=normed, sum_out=stream)
    u = up.forward(lane, normed, None)
    down.forward_fused(lane, g, pre_op=PRE_SILU_MULTIPLY, x2=u, addend=stream, out=stream)
    want = lane.read(stream, count=width)
    # two launches: gate and up stacked; the down projection reads the two halves of one output
    both = HipQuantizedMatrix.stacked(lane, [gate, up])
    assert (both.output_width, both.input_width, both.storage_bytes) == (2 * ffn, width, gate.storage_bytes + up.storage_bytes)
    stream2 = lane.allocate(width)
    launches = lane.counters()["kernel_launches"]
    gu = both.forward_fused(lane, hb, pre_op=PRE_RMS_NORM, x2=ab, norm_weight=gb, epsilon=EPS, sum_out=stream2)
    assert np.array_equal(_bits(lane.read(gu, count=ffn)), _bits(lane.read(g, count=ffn)))
    assert np.array_equal(_bits(lane.read(gu, count=ffn, offset=4 * ffn)), _bits(lane.read(u, count=ffn)))
    up_half = gu.view(4 * ffn, 4 * ffn)
    down.forward_fused(lane, gu, pre_op=PRE_SILU_MULTIPLY, x2=up_half, addend=stream2, out=stream2)
    assert lane.counters()["kernel_launches"] - launches == 2
    assert np.array_equal(_bits(lane.read(stream2, count=width)), _bits(want))
    with pytest.raises(ValueError):
        HipQuantizedMatrix.stacked(lane, [gate, down])
    for m in (gate, up, down, both):
        m.dispose()


@pytest.mark.parametrize("typ", [GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ2_S, GGML_IQ3_S, GGML_Q8_0])
def test_fused_projection_matches_separate_base_and_lora_bitwise(lane, typ):
    # the shapes, value ranges and scales of Qwen35InferenceFusedLoraTests.cs:35-63 (decode rows only)
    for in_w, out_w, rank in ((256, 5, 3), (512, 7, 8), (5120, 33, 8), (17408, 9, 3)):
        rng = np.random.default_rng(975 + in_w + typ)
        val = lambda n: rng.uniform(-0.4, 0.4, n).astype(np.float32)          # noqa: E731
        m = _matrix(typ, out_w, in_w, 6)
        m.device_payload(lane)
        x, bias, a, b = (lane.upload_raw(val(n)) for n in (in_w, out_w, rank * in_w, out_w * rank))
        z = qwen35_gpu.lora_project_a(lane, x, a, 1, in_w, rank)
        want_z = oracle.lora_a(lane.read(x, count=in_w), lane.read(a, count=rank * in_w), 1, in_w, rank)
        assert np.array_equal(_bits(lane.read(z, count=rank)), _bits(want_z.ravel()))
        for scale in (2.0, -0.75, 0.0):
            sentinel = np.full(out_w + 2, np.nan, dtype=np.float32)
            baseline, fused = lane.upload_raw(sentinel), lane.upload_raw(sentinel)
            before = lane.counters()
            m.forward(lane, x, bias, out=baseline)
            qwen35_gpu.lora_apply_b(lane, z, b, baseline, 1, out_w, rank, scale)
            m.forward_fused(lane, x, bias=bias, out=fused, lora_z=z, lora_b=b, lora_rank=rank, lora_scale=scale)
            after = lane.counters()
            assert (before["h2d_bytes"], before["d2h_bytes"], before["allocated_bytes"]) == \
                   (after["h2d_bytes"], after["d2h_bytes"], after["allocated_bytes"])
            e, g = lane.read(baseline, count=out_w + 2), lane.read(fused, count=out_w + 2)
            assert np.all(np.isfinite(g[:out_w])) and np.array_equal(_bits(e[:out_w]), _bits(g[:out_w]))
            assert np.all(np.isnan(e[out_w:])) and np.all(np.isnan(g[out_w:]))
            # the low-rank step itself against the oracle
            plain = lane.read(m.forward(lane, x, bias), count=out_w)
            want = oracle.lora_b(want_z, lane.read(b, count=out_w * rank), plain, 1, out_w, rank, scale)
            assert np.array_equal(_bits(e[:out_w]), _bits(want.ravel()))
        m.dispose()


def test_lora_argument_checks(lane):
    m = _matrix(GGML_Q4_K, 8, 256, 1)
    x, z, b = lane.allocate(256), lane.allocate(4), lane.allocate(32)
    with pytest.raises(ValueError):
        m.forward_fused(lane, x, lora_z=z, lora_b=b, lora_rank=8)           # z too small for the rank
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, lora_z=z, lora_b=b, lora_rank=0)           # buffers without a rank
    with pytest.raises(NnHipError):
        m.forward_fused(lane, x, lora_z=z, lora_b=b, lora_rank=4, lora_scale=float("inf"))
    with pytest.raises(ValueError):
        qwen35_gpu.lora_project_a(lane, x, x, 1, 256, 2)
    m.dispose()
