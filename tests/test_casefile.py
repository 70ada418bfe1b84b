"""Case files in the reference's prototxt form: the text-format reader against the one sample the
reference ships (tests/golden/parser_test.prototxt, a verbatim data file of its gtest), value
decoding (value_i / value_f / value_h hex / path / random_data), and a write -> read round trip of
a case of every operator."""
import os

import numpy as np
import pytest

import sparse_conv_oracle as oracle
from spconv_cases import out_space, random_voxels, round_to

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def casefile():
    from mluop_hip import casefile as cf
    return cf


def test_reads_the_reference_sample():
    cf = casefile()
    node, _ = cf.load(os.path.join(GOLDEN, "parser_test.prototxt"))
    assert node.get("op_name") == "abs"
    t = cf.Message(node.get("input"))
    assert t.get("id") == "input" and t.get("shape").all("dims") == [10, 10, 10, 10]
    assert t.get("layout") == "LAYOUT_ARRAY" and isinstance(t.get("layout"), cf.Enum)
    r = t.get("random_data")
    assert (r.get("seed"), r.get("upper_bound"), r.get("lower_bound"), r.get("distribution")) == \
        (23, 100, -100, "UNIFORM")
    tp = node.get("test_param")
    assert tp.all("error_func") == ["DIFF1", "DIFF2"] and tp.all("error_threshold") == [0.003, 0.003]
    assert tp.get("baseline_device") == "CPU"
    # writing it back and reading again gives the same tree
    assert cf.parse(cf.dump(node)) == node


def test_text_format_details():
    cf = casefile()
    msg = cf.parse('a: 1 b { c: -2.5 d: "x\\"y" }  # comment\n e: [1, 2, 3] f < g: true > h: 0x10 i: 1e-3 j: 2.0f')
    assert msg.get("a") == 1 and msg.get("b").get("c") == -2.5 and msg.get("b").get("d") == 'x"y'
    assert msg.all("e") == [1, 2, 3] and msg.get("f").get("g") == "true"
    assert msg.get("h") == 16 and msg.get("i") == 1e-3 and msg.get("j") == 2.0
    with pytest.raises(ValueError):
        cf.parse("a { b: 1")
    with pytest.raises(ValueError):
        cf.parse("a: 1 }")


def test_value_kinds_decode(tmp_path):
    cf = casefile()
    half = cf.CaseTensor(cf.parse(
        'id: "x" shape { dims: 3 } dtype: DTYPE_HALF value_h: "3c00" value_h: "c000" value_h: "0001"'))
    assert np.array_equal(half.values, np.array([1.0, -2.0, 2.0 ** -24], dtype=np.float32))
    single = cf.CaseTensor(cf.parse('shape { dims: 2 } dtype: DTYPE_FLOAT value_h: "3f800000" value_h: "c0490fdb"'))
    assert np.array_equal(single.values, np.array([1.0, -np.float32(np.pi)], dtype=np.float32))
    bf = cf.CaseTensor(cf.parse('shape { dims: 2 } dtype: DTYPE_BFLOAT16 value_h: "3f80" value_h: "4049"'))
    assert np.array_equal(bf.values, np.array([1.0, 3.140625], dtype=np.float32))
    ints = cf.CaseTensor(cf.parse("shape { dims: 2 dims: 2 } dtype: DTYPE_INT32 value_i: 1 value_i: -1 value_i: 7 value_i: 0"))
    assert ints.values.dtype == np.int32 and ints.values.tolist() == [[1, -1], [7, 0]]
    floats = cf.CaseTensor(cf.parse("shape { dims: 2 } dtype: DTYPE_FLOAT value_f: 0.5 value_f: -3"))
    assert floats.values.tolist() == [0.5, -3.0]
    np.arange(6, dtype=np.int32).tofile(tmp_path / "t.bin")
    frm = cf.CaseTensor(cf.parse('shape { dims: 2 dims: 3 } dtype: DTYPE_INT32 path: "t.bin"'), str(tmp_path))
    assert frm.values.tolist() == [[0, 1, 2], [3, 4, 5]]
    rnd = cf.CaseTensor(cf.parse(
        "shape { dims: 1000 } dtype: DTYPE_FLOAT random_data { seed: 3 upper_bound: 2 lower_bound: -1 distribution: UNIFORM }"))
    assert rnd.values.min() >= -1 and rnd.values.max() <= 2 and abs(rnd.values.mean() - 0.5) < 0.1
    again = cf.CaseTensor(cf.parse(
        "shape { dims: 1000 } dtype: DTYPE_FLOAT random_data { seed: 3 upper_bound: 2 lower_bound: -1 distribution: UNIFORM }"))
    assert np.array_equal(rnd.values, again.values)
    with pytest.raises(AssertionError):
        cf.CaseTensor(cf.parse("shape { dims: 1 } dtype: DTYPE_INT32 value_i: 1 value_i: 2"))


def test_value_i_of_float_tensors_holds_bit_patterns():
    """The reference's own case files store float tensors as value_i bit patterns."""
    cf = casefile()
    node, _ = cf.load(os.path.join(GOLDEN, "dynamic_point_to_voxel_forward", "case_0.prototxt"))
    assert node.get("op_name") == "dynamic_point_to_voxel_forward" and node.get("device") == "CPU"
    feats = cf.CaseTensor(node.all("input")[0])
    assert feats.values.shape == (6, 6) and feats.values.dtype == np.float32
    assert np.all(np.abs(feats.values) <= 100.0)             # drawn from U(-100, 100)
    assert feats.values[0, 0] == np.array([-1031791637], np.int32).view(np.float32)[0]
    coors = cf.CaseTensor(node.all("input")[1])
    assert coors.values.dtype == np.int32 and coors.values[3].tolist() == [-1, 18, 7]
    assert cf.criteria(node) == (["DIFF1", "DIFF2"], [0.003, 0.003])
    assert node.get("dynamic_point_to_voxel_forward_param").get("reduce_type") == "REDUCE_MODE_MEAN"
    half = cf.CaseTensor(cf.parse("shape { dims: 2 } dtype: DTYPE_HALF value_i: 15360 value_i: -16384"))
    assert half.values.tolist() == [1.0, -2.0]


def test_bf16_rounding_matches_the_oracle():
    cf = casefile()
    x = np.random.default_rng(0).standard_normal(4096).astype(np.float32)
    assert np.array_equal(cf.bf16_bits_to_f32(cf.f32_to_bf16_bits(x)), oracle.round_through_bf16(x))


def small_problem(sub_m, dtype_name, seed=5):
    rng = np.random.default_rng(seed)
    batch, space, ks, L, ci, co = 2, (6, 7, 8), (3, 3, 3), 120, 16, 32
    pad, dil = [1, 1, 1], [1, 1, 1]
    stride = [1, 1, 1] if sub_m else [2, 2, 2]
    ospace = list(space) if sub_m else out_space(space, ks, pad, stride, dil)
    idx = random_voxels(rng, batch, space, L)
    pairs, out_idx, num, n_out = oracle.get_indice_pairs(idx, batch, pad, stride, dil, ks, ospace, sub_m)
    feats = round_to(rng.standard_normal((L, ci)).astype(np.float32), dtype_name)
    w = round_to((rng.standard_normal(ks + (ci, co)) * 0.1).astype(np.float32), dtype_name)
    dy = round_to(rng.standard_normal((n_out, co)).astype(np.float32), dtype_name)
    return dict(batch=batch, space=space, ks=ks, pad=pad, stride=stride, dil=dil, ospace=ospace, idx=idx,
                pairs=pairs, out_idx=out_idx, num=num, n_out=n_out, feats=feats, w=w, dy=dy, sub_m=sub_m,
                ci=ci, co=co, L=L)


def operator_cases(c, dtype_name):
    """One case per operator, baselines from the CPU oracle."""
    cf = casefile()
    K = int(np.prod(c["ks"]))
    num = [int(v) for v in c["num"]]
    fwd = round_to(oracle.forward(c["feats"], c["w"].reshape(K, c["ci"], c["co"]), c["pairs"], num, c["n_out"]),
                   dtype_name)
    bwd = round_to(oracle.backward_data(c["dy"], c["w"].reshape(K, c["ci"], c["co"]), c["pairs"], num),
                   dtype_name)
    dw = round_to(oracle.backward_filter(c["feats"], c["dy"], c["pairs"], num), dtype_name).reshape(
        c["ks"] + (c["ci"], c["co"]))
    return [
        cf.get_indice_pairs_case(c["idx"], c["batch"], c["pad"], c["stride"], c["dil"], c["space"], c["ks"],
                                 c["ospace"], c["sub_m"], baseline=(c["out_idx"], c["pairs"], c["num"])),
        cf.indice_convolution_forward_case(c["feats"], c["w"], c["pairs"], num, c["n_out"], c["sub_m"],
                                           dtype_name, baseline=fwd),
        cf.indice_convolution_backward_data_case(c["dy"], c["w"], c["pairs"], num, c["L"], c["sub_m"],
                                                 dtype_name, baseline=bwd),
        cf.indice_convolution_backward_filter_case(c["feats"], c["dy"], c["pairs"], num, c["ks"], c["sub_m"],
                                                   dtype_name, baseline=dw),
    ]


@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_written_cases_read_back_exactly(dtype_name):
    cf = casefile()
    c = small_problem(True, dtype_name)
    for node in operator_cases(c, dtype_name):
        text = cf.dump(node)
        back = cf.parse(text)
        assert back == node
        for written, read in zip(node.all("input") + node.all("output"), back.all("input") + back.all("output")):
            t = cf.CaseTensor(read)
            assert t.values is not None and list(t.values.shape) == t.shape
    fwd = operator_cases(c, dtype_name)[1]
    feats = cf.CaseTensor(fwd.all("input")[0])
    assert np.array_equal(feats.values, c["feats"])          # value_h carries the exact bits
    p = fwd.get("indice_convolution_forward_param")
    assert p.all("indice_num") == [int(v) for v in c["num"]] and p.get("num_active_out") == c["n_out"]
    gp = operator_cases(c, dtype_name)[0].get("get_indice_pairs_param")
    assert gp.all("filter_space") == [3, 3, 3] and gp.get("sub_m") == 1 and gp.get("batch") == 2


@pytest.mark.gpu
@pytest.mark.parametrize("sub_m", [True, False])
@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
def test_replayed_cases_meet_their_thresholds(gpu_handle, tmp_path, sub_m, dtype_name):
    """Cases written to disk with oracle baselines, replayed through the C API from the files."""
    cf = casefile()
    c = small_problem(sub_m, dtype_name, seed=6)
    thr = 1e-5 if dtype_name == "float32" else 3e-3
    for node in operator_cases(c, dtype_name):
        tp = node.get("test_param")
        if node.get("op_name") != "get_indice_pairs":
            tp[:] = [(n, (thr if n == "error_threshold" else v)) for n, v in tp]
        path = tmp_path / (node.get("op_name") + ".prototxt")
        path.write_text(cf.dump(node))
        res = cf.replay(str(path), gpu_handle)
        assert res.errors, "no baseline compared"
        assert res.passed, (node.get("op_name"), res.errors)


@pytest.mark.gpu
def test_replay_refuses_other_operators(gpu_handle):
    cf = casefile()
    with open(os.path.join(GOLDEN, "parser_test.prototxt")) as f:
        text = f.read()
    with pytest.raises(ValueError):
        cf.replay(text, gpu_handle)


REFERENCE_BWD_DATA_CASE = os.path.join(GOLDEN, "indice_convolution_backward_data", "case_0.prototxt")


def reference_backward_data_case():
    """The one sparse-convolution case the reference keeps in its tree
    (zoo/indice_convolution_backward_data/test_case/case_0.prototxt, a verbatim data file): explicit
    pairs, seeded random out_grad and filter (filled by this module's own generator: the reference
    generator's bit stream is not reproduced), no stored baseline."""
    cf = casefile()
    node, base = cf.load(REFERENCE_BWD_DATA_CASE)
    ins = [cf.CaseTensor(t, base) for t in node.all("input")]
    out = cf.CaseTensor(node.all("output")[0], base)
    return node, ins, out


def test_reference_backward_data_case_reads():
    cf = casefile()
    node, (dy, w, pairs), out = reference_backward_data_case()
    assert node.get("op_name") == "indice_convolution_backward_data"
    assert dy.values.shape == (10, 100) and w.values.shape == (3, 3, 210, 100) and w.layout == 2  # HWCN
    assert pairs.values.shape == (9, 2, 10) and pairs.values.dtype == np.int32
    assert all(pairs.values[k, c].tolist() == list(range(10)) for k in range(9) for c in range(2))
    assert list(out.shape) == [10, 210] and out.values is None
    p = node.get("indice_convolution_backward_data_param")
    assert p.all("indice_num") == [10] * 9 and p.get("inverse") == 0 and p.get("sub_m") == 0
    assert cf.criteria(node) == (["DIFF1", "DIFF2"], [1e-5, 1e-5])
    assert np.abs(dy.values).max() <= 1.0 and np.abs(w.values).max() <= 1.0   # U(-1, 1) as the file asks
    # identity pairs at every offset: the operator reduces to one dense product with the summed filter
    ref = oracle.backward_data(dy.values, w.values.reshape(9, 210, 100), pairs.values, [10] * 9)
    dense = dy.values.astype(np.float64) @ w.values.astype(np.float64).sum(axis=(0, 1)).T
    np.testing.assert_allclose(ref, dense, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_reference_backward_data_case_replays(gpu_handle):
    """Replayed through the C API from the file itself and graded at the file's own thresholds
    against the oracle on the same generated inputs."""
    cf = casefile()
    node, (dy, w, pairs), out = reference_backward_data_case()
    res = cf.replay(REFERENCE_BWD_DATA_CASE, gpu_handle)
    got = res.outputs["in_grad"]
    assert got.shape == (10, 210)
    ref = oracle.backward_data(dy.values, w.values.reshape(9, 210, 100), pairs.values, [10] * 9)
    funcs, thresholds = cf.criteria(node)
    assert cf.diff1(got, ref) <= thresholds[0] and cf.diff2(got, ref) <= thresholds[1]


# ---- the three operators upstream of the sparse convolutions ---------------------------------

def test_fewer_values_than_elements_are_padded_with_zeros():
    """The reference's backward case lists 150 values for a [34, 5] tensor (parser.cpp:371-383 takes
    the count from the list and warns)."""
    cf = casefile()
    t = cf.CaseTensor(cf.parse("shape { dims: 2 dims: 3 } dtype: DTYPE_INT32 value_i: 4 value_i: 5 value_i: 6 value_i: 7"))
    assert t.values.tolist() == [[4, 5, 6], [7, 0, 0]]
    node, _ = cf.load(os.path.join(GOLDEN, "dynamic_point_to_voxel_backward", "case_1.prototxt"))
    grad = cf.CaseTensor(node.all("input")[0])
    assert grad.values.shape == (34, 5) and len(node.all("input")[0].all("value_i")) == 150
    assert np.all(grad.values[30:] == 0) and np.any(grad.values[29] != 0)
    with pytest.raises(AssertionError):
        cf.CaseTensor(cf.parse("shape { dims: 1 } dtype: DTYPE_INT32 value_i: 4 value_i: 5"))


def test_diff3_is_the_largest_relative_error():
    cf = casefile()
    want = np.array([1.0, -2.0, 0.0, 4.0], np.float32)
    assert cf.diff3(want, want) == 0.0
    got = want * np.float32(1.01)
    assert abs(cf.diff3(got, want) - 0.01) < 1e-6
    # where the baseline is (nearly) zero the absolute error counts
    assert abs(cf.diff3(np.array([0.5], np.float32), np.array([0.0], np.float32)) - 0.5) < 1e-12
    assert abs(cf.diff3(np.array([5e-5], np.float32), np.array([2e-5], np.float32), "float16") - 3e-5) < 1e-9
    assert cf.diff3(np.array([5e-5], np.float32), np.array([2e-5], np.float32), "float32") > 1.4
    import sparse_conv_oracle as oracle
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    assert abs(cf.diff3(a, b) - oracle.diff3(a, b)) <= 1e-9 * oracle.diff3(a, b)


def test_written_upstream_cases_read_back_exactly():
    import dynamic_point_to_voxel_oracle as dpv
    import voxelization_oracle as vox
    cf = casefile()
    rng = np.random.default_rng(5)
    pts = rng.uniform(-1, 5, (200, 4)).astype(np.float32)
    vs, cr = [0.5, 0.5, 1.0], [0.0, 0.0, 0.0, 4.0, 4.0, 2.0]
    want = vox.voxelization(pts, vs, cr, 5, 40)
    node = cf.parse(cf.dump(cf.voxelization_case(pts, vs, cr, 5, 40, baseline=want)))
    assert node.get("op_name") == "voxelization"
    p = node.get("voxelization_param")
    assert (p.get("max_points"), p.get("max_voxels"), p.get("ndim"), p.get("deterministic")) == (5, 40, 3, "true")
    ins = [cf.CaseTensor(t).values for t in node.all("input")]
    assert np.array_equal(ins[0], pts) and ins[1].tolist() == vs and ins[2].tolist() == cr
    for t, w in zip(node.all("output"), want):
        assert np.array_equal(cf.CaseTensor(t).values.reshape(-1), np.asarray(w).reshape(-1), equal_nan=True)

    feats = rng.uniform(-100, 100, (50, 3)).astype(np.float32)
    coors = rng.integers(-1, 4, (50, 3)).astype(np.int32)
    fwd = dpv.forward("max", feats, coors)
    node = cf.parse(cf.dump(cf.dynamic_point_to_voxel_forward_case(feats, coors, "max", baseline=fwd[:5])))
    assert node.get("dynamic_point_to_voxel_forward_param").get("reduce_type") == "REDUCE_MODE_MAX"
    assert len(node.all("input")) == 2 and len(node.all("output")) == 5
    assert np.array_equal(cf.CaseTensor(node.all("output")[0]).values, fwd[0])
    assert cf.CaseTensor(node.all("output")[4]).values.tolist() == [fwd[4]]

    g = rng.standard_normal((50, 3)).astype(np.float32)
    bwd = dpv.backward(g, feats, fwd[0], fwd[2], fwd[4])
    node = cf.parse(cf.dump(cf.dynamic_point_to_voxel_backward_case(g, feats, fwd[0], fwd[2], fwd[3], fwd[4],
                                                                    baseline=bwd)))
    assert len(node.all("input")) == 6 and node.get("dynamic_point_to_voxel_backward_param") is not None
    assert np.array_equal(cf.CaseTensor(node.all("output")[0]).values, bwd)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["dynamic_point_to_voxel_forward/case_0.prototxt",
                                  "dynamic_point_to_voxel_forward/case_1.prototxt",
                                  "dynamic_point_to_voxel_backward/case_1.prototxt"])
def test_reference_upstream_cases_replay(gpu_handle, name):
    """The reference's own case files with their stored baselines, through `replay` as they are.
    Integer outputs and the backward gradient (copies of input values) must come out exact; the
    forward features within the file's thresholds and, being sums in point order, within 1e-6."""
    cf = casefile()
    res = cf.replay(os.path.join(GOLDEN, name), gpu_handle)
    assert res.passed, res.errors
    assert len(res.errors) >= 1      # the backward case names one measure (DIFF3, threshold 0)
    for tid, func, err, thr in res.errors:
        assert err <= 1e-6, (tid, func, err)


@pytest.mark.gpu
def test_written_upstream_cases_replay(gpu_handle, tmp_path):
    import dynamic_point_to_voxel_oracle as dpv
    import voxelization_oracle as vox
    cf = casefile()
    rng = np.random.default_rng(6)
    pts = rng.uniform(-1, 5, (3000, 4)).astype(np.float32)
    vs, cr = [0.5, 0.5, 1.0], [0.0, 0.0, 0.0, 4.0, 4.0, 2.0]
    path = tmp_path / "vox.prototxt"
    path.write_text(cf.dump(cf.voxelization_case(pts, vs, cr, 5, 40, baseline=vox.voxelization(pts, vs, cr, 5, 40))))
    res = cf.replay(str(path), gpu_handle)
    assert res.passed and len(res.errors) == 8 and all(e[2] == 0.0 for e in res.errors), res.errors

    feats = rng.uniform(-100, 100, (2000, 5)).astype(np.float32)
    coors = rng.integers(-1, 9, (2000, 3)).astype(np.int32)
    for mode in ("max", "mean"):
        fwd = dpv.forward(mode, feats, coors.copy())
        res = cf.replay(cf.dump(cf.dynamic_point_to_voxel_forward_case(feats, coors, mode, baseline=fwd[:5])),
                        gpu_handle)
        assert res.passed and len(res.errors) == 10 and all(e[2] == 0.0 for e in res.errors), res.errors
    fwd = dpv.forward("max", feats, coors.copy())
    g = rng.standard_normal((2000, 5)).astype(np.float32)
    bwd = dpv.backward(g, feats, fwd[0], fwd[2], fwd[4])
    res = cf.replay(cf.dump(cf.dynamic_point_to_voxel_backward_case(g, feats, fwd[0], fwd[2], fwd[3], fwd[4],
                                                                    baseline=bwd)), gpu_handle)
    assert res.passed and all(e[2] == 0.0 for e in res.errors), res.errors
