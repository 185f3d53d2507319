"""The order of the parameters inside the reference's w8a32 weight blobs
(arg0-w8a32-f32.data / arg0-w8a32-i8.data), derived from the reference's own
text and held against the one table the blob reader cuts the blobs by
(buddy_hip_w8a32_blob_layout).

What the text fixes:
  * the parameters in trace order: the arguments of
    examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:4 without the
    run-time inputs (i64 token / positions, rank-4 KV caches);
  * packing walks them in that order with one running element offset per dtype
    (frontend/Python/graph/graph.py:848-863 builds one pack per dtype,
    :1001-1018 advances `_current_param_pack_offset[dtype]` per placeholder);
  * the weight of a plain matmul becomes int8, the weight of a matmul + bias
    (AddMM: q/k/v) stays f32
    (frontend/Python/graph/transform/quantization/weight_only_channel_wise.py:366-461);
  * one f32 scaler per int8 weight (one value per output channel) is appended
    after all original parameters, sorted by the position of its weight
    (frontend/Python/graph/transform/quantization/quantize.py:561-590).
The argument list is kept as data in tests/golden/decode_graph_params.json
(written by tests/golden/make_decode_graph_params.py); where the reference tree
is present the fixture is re-derived from the text and compared.

This pins the layout to the reference's text, not to a blob written by the
reference importer: parity of the order is still unpinned by execution.
"""
import ctypes
import json
import sys
from pathlib import Path

import pytest

from buddy_mlir_amd.session import QWEN2_1P5B

GOLDEN = Path(__file__).resolve().parent / "golden"
F32, I8 = 0, 1
(EMBED, INV_FREQ, LN1, Q_BIAS, Q_W, K_BIAS, K_W, V_BIAS, V_W, O_W, LN2, GATE_W, UP_W,
 DOWN_W, LN_F, LM_HEAD_W, O_SCALE, GATE_SCALE, UP_SCALE, DOWN_SCALE, LM_HEAD_SCALE) = range(21)


class BlobEntry(ctypes.Structure):
    _fields_ = [("param", ctypes.c_int32), ("layer", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64),
                ("offset", ctypes.c_int64), ("count", ctypes.c_int64)]


def library_table(bh, shape):
    cs = shape.c()
    n = bh.buddy_hip_w8a32_blob_layout(ctypes.byref(cs), None, 0)
    assert n > 0
    buf = (BlobEntry * n)()
    assert bh.buddy_hip_w8a32_blob_layout(ctypes.byref(cs), buf, n) == n
    return list(buf)


def graph_args():
    return json.loads((GOLDEN / "decode_graph_params.json").read_text())["args"]


def layout_from_text(args):
    """[(dtype, offset, shape, arg index or ('scaler', arg index))] in blob order."""
    params = [a for a in args if a["dtype"] == "f32" and len(a["shape"]) <= 2]
    inputs = [a for a in args if a not in params]
    assert all(a["dtype"] == "i64" or len(a["shape"]) == 4 for a in inputs)
    off = {F32: 0, I8: 0}
    out, quantized = [], []
    for a in params:
        dt = I8 if a["use"] == "matmul" else F32
        n = 1
        for d in a["shape"]:
            n *= d
        out.append((dt, off[dt], tuple(a["shape"]), a["arg"]))
        off[dt] += n
        if dt == I8:
            quantized.append(a)
    for a in quantized:  # scalers: after every original parameter, in weight order
        n = a["shape"][1]
        out.append((F32, off[F32], (n,), ("scaler", a["arg"])))
        off[F32] += n
    return out, off


def test_fixture_matches_the_reference_text():
    ref = Path("/root/reference/examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir")
    if not ref.exists():
        pytest.skip("reference tree not present")
    sys.path.insert(0, str(GOLDEN))
    import make_decode_graph_params as gen
    assert gen.parse(ref.read_text()) == graph_args()


def test_text_gives_the_reference_size_constants():
    """F32ParamsSize / I8ParamsSize of
    examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:32-33."""
    _, off = layout_from_text(graph_args())
    assert off[F32] == 322338752 and off[I8] == 1455489024


def test_reader_table_follows_the_text(bh):
    want, off = layout_from_text(graph_args())
    got = library_table(bh, QWEN2_1P5B)
    assert len(got) == len(want)
    for e, (dt, offset, shape, _) in zip(got, want):
        eshape = (e.cols,) if len(shape) == 1 else (e.rows, e.cols)
        assert (e.dtype, e.offset, eshape, e.count) == (dt, offset, shape, e.rows * e.cols), \
            (e.param, e.layer)
    n_f32, n_i8 = ctypes.c_int64(), ctypes.c_int64()
    cs = QWEN2_1P5B.c()
    bh.buddy_hip_w8a32_blob_sizes(ctypes.byref(cs), ctypes.byref(n_f32), ctypes.byref(n_i8))
    assert (n_f32.value, n_i8.value) == (off[F32], off[I8])


def test_reader_names_agree_with_how_the_graph_uses_each_argument(bh):
    """The table's parameter names against the use the graph's body makes of the
    argument at the same place: biases are the vectors added to the result of the
    matmul whose weight follows them, q/k/v weights are the AddMM weights, the
    int8 entries are exactly the plain-matmul weights, every scaler belongs to
    the int8 weight at the same rank."""
    args = graph_args()
    want, _ = layout_from_text(args)
    got = library_table(bh, QWEN2_1P5B)
    by_arg = {a["arg"]: a for a in args}
    bias_of = {a["bias"]: a["arg"] for a in args if a["use"] == "addmm"}
    int8_weights = []
    for e, (dt, _, _, src) in zip(got, want):
        if isinstance(src, tuple):
            continue
        a = by_arg[src]
        if e.param in (Q_BIAS, K_BIAS, V_BIAS):
            assert src in bias_of and bias_of[src] == src + 1
        elif e.param in (Q_W, K_W, V_W):
            assert a["use"] == "addmm" and a["bias"] == src - 1
        elif e.param in (O_W, GATE_W, UP_W, DOWN_W, LM_HEAD_W):
            assert a["use"] == "matmul" and e.dtype == I8
            int8_weights.append(e)
        else:
            assert a["use"] is None and e.dtype == F32, (e.param, src)
            assert src not in bias_of
    scalers = [e for e in got if e.param >= O_SCALE]
    assert len(scalers) == len(int8_weights) == 4 * QWEN2_1P5B.layers + 1
    pair = {O_W: O_SCALE, GATE_W: GATE_SCALE, UP_W: UP_SCALE, DOWN_W: DOWN_SCALE,
            LM_HEAD_W: LM_HEAD_SCALE}
    for w, s in zip(int8_weights, scalers):
        assert (pair[w.param], w.layer, w.cols) == (s.param, s.layer, s.cols)
    # the layer pattern: embed, inv_freq, 28 x 12 parameters, ln_f, lm_head
    names = [e.param for e in got if e.param < O_SCALE]
    per_layer = [LN1, Q_BIAS, Q_W, K_BIAS, K_W, V_BIAS, V_W, O_W, LN2, GATE_W, UP_W, DOWN_W]
    assert names == [EMBED, INV_FREQ] + per_layer * QWEN2_1P5B.layers + [LN_F, LM_HEAD_W]
