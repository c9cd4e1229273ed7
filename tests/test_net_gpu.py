"""GPU: the C++ bnn::Net on .dab models vs the CPU restatement of the layer loop.

Bit-exact wherever the data is integer (packed activations, raw BinConv
counts), 1e-4 relative after float layers (north_star tolerance)."""
import numpy as np
import pytest

import oracle as orc
from oracle import net as orc_net

pytestmark = pytest.mark.gpu

RTOL = 1e-4


@pytest.fixture(scope="module")
def mods():
    import torch
    assert torch.cuda.is_available()
    from dabnn_amd import dab_format, models, net
    return dab_format, models, net


def close(got, want):
    scale = max(np.abs(want).max(), 1e-6)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * scale)


def blobs_not_produced(n, layers):
    """Output names of the model whose blob the optimized layer list does not write (get_blob says so)."""
    gone = set()
    for layer in layers:
        try:
            n.blob_info(layer["output"])
        except RuntimeError as e:
            assert "is not produced" in str(e), str(e)
            gone.add(layer["output"])
    return gone


def check_every_segment(n, layers, inits, image, absent=()):
    """Every layer group of the device run against the CPU restatement fed with the device's own input blobs:
    bit-exact after a binary convolution (counts are integers; Affine and Add round alike on both sides) and for
    max pooling, 1e-4 relative after float convolutions and average pooling."""
    checked = 0
    for name, first_type, want in orc_net.run_segments(layers, inits, lambda b: n.get_blob(b)[image], absent):
        got = n.get_blob(name)[image]
        if first_type in ("BinConv2D", "MaxPool", "Affine", "Add", "Relu", "PRelu", "Concat"):
            np.testing.assert_array_equal(got, want, err_msg=name)
        else:
            close(got, want)
        checked += 1
    return checked


def check_packed_inputs(n, layers, image):
    """The packed input every direct BinConv worked on is pack_mat of the fp32 blob it reads, whether the layer packed
    it itself or the previous block's fused pass wrote it."""
    checked = 0
    descs = [d for d in n.layers() if d.startswith("Bin Conv")]
    convs = [l for l in layers if l["type"] == "BinConv2D"]
    assert len(descs) == len(convs)
    for layer, desc in zip(convs, descs):
        if "DIRECT_CONV" not in desc:
            continue
        packed = n.get_blob("binaized_for_%s_cal" % layer["output"])[image]
        np.testing.assert_array_equal(packed, orc.pack_mat(n.get_blob(layer["input"])[image]), err_msg=layer["name"])
        checked += 1
    return checked


def drift_ok(got, want):
    """End to end only a loose bound holds: one flipped sign early on moves the logits by about a percent."""
    assert np.corrcoef(got.ravel(), want.ravel())[0, 1] > 0.98


def test_small_net_matches_cpu_layer_loop(mods):
    df, models, net = mods
    layers, inits, inputs = models.small_bnn(1, hw=16, width=64)
    buf = df.write_model(layers, inits, inputs)
    batch = 3
    x = np.random.default_rng(5).standard_normal((batch, 16, 16, 3)).astype(np.float32)
    n = net.Net(batch=batch).read_buf(buf)
    descs = n.layers()
    assert sum("DIRECT_CONV" in d for d in descs) == 3 and sum("BGEMM" in d for d in descs) == 1
    n.run(x)
    logits = n.get_blob("logits").reshape(batch, -1)
    for i in range(batch):
        assert check_every_segment(n, layers, inits, i) == 7
        cpu = orc_net.run_model(layers, inits, x[i])
        drift_ok(logits[i], cpu["logits"])
        # packed input of every BinConv: bit-exact unless a float sits within rounding of zero
        for blk in ("b0", "b1", "b2"):
            packed = n.get_blob("binaized_for_%s_cnt_cal" % blk)[i]
            src = {"b0": "conv1_out", "b1": "b0_out", "b2": "b1_bn"}[blk]
            assert packed.shape == orc.pack_mat(cpu[src]).shape
    n.close()


def test_dense_net_with_concat_and_prelu_matches_cpu_layer_loop(mods):
    """A BiDenseNet-style graph: Concat joins each binary convolution's result to its input features, PRelu (one slope
    and one per channel) follows the float convolutions, and the binary convolutions see 64/128/192 channels."""
    df, models, net = mods
    layers, inits, inputs = models.dense_bnn(3, hw=16)
    batch = 2
    x = np.random.default_rng(9).standard_normal((batch, 16, 16, 3)).astype(np.float32)
    n = net.Net(batch=batch).read_buf(df.write_model(layers, inits, inputs))
    descs = n.layers()
    assert sum(d.startswith("Concat") for d in descs) == 5 and sum(d.startswith("PRelu") for d in descs) == 2
    assert sum("DIRECT_CONV" in d for d in descs) == 3 and sum("BGEMM" in d for d in descs) == 2
    n.run(x)
    logits = n.get_blob("logits").reshape(batch, -1)
    for i in range(batch):
        assert check_every_segment(n, layers, inits, i) == 15
        assert check_packed_inputs(n, layers, i) == 3
        drift_ok(logits[i], orc_net.run_model(layers, inits, x[i])["logits"])
    assert n.get_blob("d1l2_cat").shape == (batch, 16, 16, 256)
    n.close()


def test_binconv_counts_inside_net_are_bit_exact(mods):
    """One BinConv + Affine net: the blob holds raw counts before the affine when the affine is identity-free;
    here the net is cut after the BinConv so the counts themselves are the output."""
    df, models, net = mods
    r = np.random.default_rng(7)
    for (c, cout, k, stride, pad) in [(64, 64, 3, 1, 1), (128, 64, 3, 2, 1), (192, 24, 3, 1, 1), (128, 16, 5, 2, 2),
                                      (64, 12, 1, 1, 0)]:
        wf = r.standard_normal((cout, k, k, c)).astype(np.float32)
        inits = [{"name": "w", "shape": [cout, k, k, c], "data": models.pack_weight(wf).ravel(),
                  "align_hwc_to_128": c != 64}]
        layers = [{"type": "BinConv2D", "name": "bc", "input": "data", "weight": "w", "output": "cnt",
                   "pads": [pad] * 4, "strides": [stride, stride], "dilations": [1, 1]}]
        x = r.standard_normal((2, 12, 12, c)).astype(np.float32)
        for optimize in (True, False):
            n = net.Net(batch=2, optimize=optimize).read_buf(df.write_model(layers, inits, [("data", [1, 12, 12, c])]))
            n.run(x)
            got = n.get_blob("cnt")
            for i in range(2):
                want = orc_net.run_model(layers, inits, x[i])["cnt"]
                np.testing.assert_array_equal(got[i], want)
            n.close()


def test_optimize_flag_gives_identical_outputs(mods):
    """tests/net_test.cpp:29-50: optimize=false and optimize=true agree."""
    df, models, net = mods
    layers, inits, inputs = models.small_bnn(2, hw=16, width=64)
    buf = df.write_model(layers, inits, inputs)
    x = np.random.default_rng(6).standard_normal((2, 16, 16, 3)).astype(np.float32)
    outs = []
    for optimize in (True, False):
        n = net.Net(batch=2, optimize=optimize).read_buf(buf)
        if not optimize:
            assert all("DIRECT_CONV" not in d for d in n.layers())
        n.run(x)
        outs.append(n.get_blob("logits").copy())
        n.close()
    np.testing.assert_array_equal(outs[0], outs[1])


@pytest.mark.parametrize("batch", [1, 2])
@pytest.mark.parametrize("stem", [False, True])
def test_bireal18_batch2_matches_cpu(mods, tmp_path, stem, batch):
    """Bi-Real-18 as the benchmark runs it at batch 1 (and at 2, the same kernels on two images)."""
    df, models, net = mods
    layers, inits, inputs = models.bireal18(11, stem=stem)
    path = tmp_path / "bireal18.dab"
    path.write_bytes(df.write_model(layers, inits, inputs))
    x = np.random.default_rng(8).standard_normal((batch, 224, 224, 3)).astype(np.float32)
    n = net.Net(batch=batch).read(str(path))
    assert sum("Bin Conv" in d for d in n.layers()) == 16
    n.run(x)
    logits = n.get_blob("logits").reshape(batch, -1)
    assert logits.shape == (batch, 1000)
    descs = n.layers()
    # the max pool and every block hand their successor the packed input (at this batch the blocks with 512 input
    # channels run the small-problem kernel, whose work items are whole bytes of sign bits); the three Adds of the
    # down-sampling blocks are fused too, behind their shortcut branch
    assert sum("+ Sign" in d for d in descs) == 15 and sum("packed input from its producer" in d for d in descs) == 16
    assert sum("+ Affine + Add" in d for d in descs) == 16 and not any(d.startswith("Add") for d in descs)
    # the three shortcut branches pool inside their 1x1 convolution, and at this batch the classifier does too
    assert sum("AvePool 2x2 of" in d for d in descs) == 3 and not any(d.startswith("AvePool") for d in descs)
    assert sum("AvePool over all of 7x7 inside" in d for d in descs) == 1
    # the pooled blobs of the three shortcut branches have no other reader and are not written
    gone = blobs_not_produced(n, layers)
    assert gone == {"s%db0_sc_pool_out" % s for s in (2, 3, 4)}
    with pytest.raises(RuntimeError, match="is not produced: the AvePool runs inside the convolution"):
        n.get_blob("s2b0_sc_pool_out")
    for i in range(batch):
        assert check_every_segment(n, layers, inits, i, gone) >= 17
        assert check_packed_inputs(n, layers, i) == 16
    cpu = orc_net.run_model(layers, inits, x[0])
    drift_ok(logits[0], cpu["logits"])
    n.set_profile(True)
    n.run(x)
    report = n.time_report()
    assert "Bin Conv" in report and "Float Conv" in report and "total" in report
    n.close()
    # at a large batch the two producers with 512 input channels leave the packing to their successors (the unit
    # kernel's work items of four units make the sign bits dearer than a separate pass there) ...
    large = net.Net(batch=256).read(str(path))
    descs = large.layers()
    assert sum("+ Sign" in d for d in descs if d.startswith("Bin Conv")) == 13
    assert sum("packed input from its producer" in d for d in descs) == 14
    large.close()
    # ... and write them themselves at the sizes the row-split kernel takes
    big = net.Net(batch=64).read(str(path))
    descs = big.layers()
    assert sum("+ Sign" in d for d in descs if d.startswith("Bin Conv")) == 15
    assert sum("packed input from its producer" in d for d in descs) == 16
    # and either stem's last convolution runs with its MaxPool inside (the three-convolution stem's on the
    # split-operand kernel at this size, which pools a tile column's rows and columns in registers)
    assert sum("+ MaxPool 3x3 stride 2 + Sign" in d for d in descs) == 1
    assert not any(d.startswith("MaxPool") for d in descs)
    # and the global pool is a launch of its own before the classifier's matrix product
    assert sum(d.startswith("AvePool") for d in descs) == 1 and not any("AvePool over all" in d for d in descs)
    big.close()


@pytest.mark.parametrize("stem", [False, True])
def test_bireal18_stem_and_maxpool_in_one_pass(mods, stem):
    """From a handful of images on (7x7 stem) or whenever the bands fill whole rounds of blocks and the problem is too
    small for the split-operand kernel (the 3x3 stem: batch 18) the last float convolution of the stem and the MaxPool
    behind it run as one pass that
    never writes the convolution's blob: the pooled blob and the packed copy still match the CPU layers fed with the
    device's own input, the elided blob is reported as such, and optimize = false brings it back."""
    df, models, net = mods
    layers, inits, inputs = models.bireal18(12, stem=stem)
    buf = df.write_model(layers, inits, inputs)
    batch = 18 if stem else 40
    x = np.random.default_rng(10).standard_normal((batch, 224, 224, 3)).astype(np.float32)
    n = net.Net(batch=batch).read_buf(buf)
    descs = n.layers()
    assert sum("+ MaxPool 3x3 stride 2 + Sign" in d for d in descs) == 1 and not any(d.startswith("MaxPool") for d in descs)
    gone = blobs_not_produced(n, layers)
    last_conv = "stem2_out" if stem else "conv1_out"
    shortcut_pools = {"s%db0_sc_pool_out" % s for s in (2, 3, 4)}  # pooled inside the convolutions that read them
    assert gone == {last_conv, last_conv + "_bn"} | ({last_conv + "_bn_relu"} if stem else set()) | shortcut_pools
    with pytest.raises(RuntimeError, match="is not produced: the convolution and the MaxPool"):
        n.get_blob(last_conv)
    n.run(x)
    for i in (0, batch - 1):
        assert check_every_segment(n, layers, inits, i, gone) >= 16
        assert check_packed_inputs(n, layers, i) == 16
    pooled = n.get_blob("pool1_out").copy()
    n.close()
    plain = net.Net(batch=batch, optimize=False).read_buf(buf)
    assert blobs_not_produced(plain, layers) == set()
    plain.run(x)
    conv = plain.get_blob(last_conv)  # after the in-place Affine (and Relu)
    for i in (0, 11, batch - 1):
        want = orc.max_pool(conv[i], 3, 3, 1, 1, 2, 2)
        close(pooled[i], want)
    plain.close()


class CachedBlobs:
    """A Net whose get_blob copies each blob from the device once: at batch 256 a blob is up to 205 MB and the segment
    checks ask for the same ones many times."""

    def __init__(self, n):
        self.n, self.cache = n, {}

    def get_blob(self, name):
        if name not in self.cache:
            self.cache[name] = self.n.get_blob(name)
        return self.cache[name]

    def __getattr__(self, attr):
        return getattr(self.n, attr)


@pytest.mark.parametrize("seed", range(3))
def test_miniature_nets_on_random_sizes(mods, seed):
    """The two miniature graphs at seeded random image sizes and batches: every layer group of the first and the last
    image against the CPU layers, packed inputs, and the same logits from a second run and from the graph."""
    import torch
    df, models, net = mods
    r = np.random.default_rng(500 + seed)
    for _ in range(6):
        hw, batch = int(r.choice([8, 12, 16, 20, 24, 32])), int(r.integers(1, 70))
        dense = bool(r.integers(0, 2))
        make = models.dense_bnn if dense else models.small_bnn
        layers, inits, inputs = make(int(r.integers(0, 1000)), hw=hw)
        case = "%s hw %d batch %d" % ("dense" if dense else "small", hw, batch)
        n = net.Net(batch=batch).read_buf(df.write_model(layers, inits, inputs))
        gone = blobs_not_produced(n, layers)
        x = torch.randn((batch, hw, hw, 3), generator=torch.Generator().manual_seed(batch)).cuda()
        n.run(x)
        for i in sorted({0, batch - 1}):
            assert check_every_segment(n, layers, inits, i, gone) >= 7, case
            assert check_packed_inputs(n, layers, i) == 3, case
        first = n.get_blob("logits").copy()
        n.run(x)
        n.run(x)
        np.testing.assert_array_equal(n.get_blob("logits"), first, err_msg=case)
        n.close()


@pytest.mark.parametrize("stem", [False, True])
def test_bireal18_batches_between_the_benchmarks_match_cpu(mods, stem):
    """Which kernel runs a layer changes with the batch (the depth-splitting kernel for small problems, the one-pass
    stem from a handful of images on, the split-operand convolutions over 32 channels from batch 21, the second builds
    of the unit kernel): batch sizes on both sides of those switches, every layer group of the first and the last image
    against the CPU layers fed with the device's own blobs, and the same logits from a second run and from the graph."""
    import torch
    df, models, net = mods
    layers, inits, inputs = models.bireal18(31, stem=stem)
    buf = df.write_model(layers, inits, inputs)
    for batch in (3, 5, 9, 17, 20, 21, 33, 100, 168):
        n = net.Net(batch=batch).read_buf(buf)
        gone = blobs_not_produced(n, layers)
        x = torch.randn((batch, 224, 224, 3), generator=torch.Generator().manual_seed(batch)).cuda()
        n.run(x)
        cached = CachedBlobs(n)
        for i in (0, batch - 1):
            assert check_every_segment(cached, layers, inits, i, gone) >= 19, batch
            assert check_packed_inputs(cached, layers, i) == 16, batch
        first = cached.get_blob("logits").copy()
        n.run(x)
        n.run(x)
        np.testing.assert_array_equal(n.get_blob("logits"), first, err_msg="batch %d" % batch)
        n.close()
        del x
        torch.cuda.empty_cache()


@pytest.mark.parametrize("stem", [False, True])
def test_bireal18_batch256_matches_cpu(mods, stem):
    """The benchmark's throughput configuration, both stems: at batch 256 other kernels run than at batch 2 or 64 (the
    four-waves-per-SIMD builds of the direct convolution with their epilogues, 64 x 256 tiles in the pooled shortcut
    convolutions, the one-pass stem without a carry launch, blocks with 512 input channels that leave the packing to
    their successor).  Every layer group of nine images spread over the batch against the CPU layers fed with the
    device's own blobs, and every packed BinConv input against pack_mat of the blob it stands for."""
    import torch
    df, models, net = mods
    from dabnn_amd import capi
    layers, inits, inputs = models.bireal18(14, stem=stem)
    batch = 256
    n = net.Net(batch=batch).read_buf(df.write_model(layers, inits, inputs))
    descs = n.layers()
    assert sum("Bin Conv" in d for d in descs) == 16
    assert sum("+ MaxPool 3x3 stride 2 + Sign" in d for d in descs) == 1
    assert not any(d.startswith("MaxPool") for d in descs)
    # the builds this configuration is there to cover
    assert capi.lib.dab_bconv3x3_build(batch * 56 * 56, 64, 64) == 2
    assert capi.lib.dab_bconv3x3_build(batch * 28 * 28, 128, 128) == 2
    assert capi.lib.dab_bconv3x3_build(batch * 14 * 14, 256, 256) == 2
    assert capi.lib.dab_bconv3x3_build(batch * 7 * 7, 512, 512) == 2
    assert capi.lib.dab_bconv3x3_build(batch * 7 * 7, 256, 512) == 1
    gone = blobs_not_produced(n, layers)
    gen = torch.Generator().manual_seed(21)
    x = torch.randn((batch, 224, 224, 3), generator=gen).cuda()
    n.run(x)
    cached = CachedBlobs(n)
    # images spread over the batch: a tile-indexing fault in the middle of a launch must not hide between the ends
    for i in (0, 31, 63, 100, 127, 128, 191, 222, batch - 1):
        assert check_every_segment(cached, layers, inits, i, gone) >= 19, i
        assert check_packed_inputs(cached, layers, i) == 16, i
    first = cached.get_blob("logits").reshape(batch, -1).copy()
    cached.cache.clear()
    # a second and a third run (the third is the captured graph) give the same logits
    n.run(x)
    n.run(x)
    np.testing.assert_array_equal(n.get_blob("logits").reshape(batch, -1), first)
    drift_ok(first[0], orc_net.run_model(layers, inits, x[0].cpu().numpy())["logits"])
    n.close()


def test_binconv_over_1024_channels_direct_equals_bgemm(mods):
    """A binary convolution over 1024 channels takes the direct kernel (two passes over 512 channels each) when the net
    optimizes and im2col + bgemm when it does not: the same blobs, and the CPU layers agree group by group; the Affine
    behind it stays a layer of its own (no fused epilogue for this depth)."""
    df, models, net = mods
    r = np.random.default_rng(17)
    w1 = (r.standard_normal((1024, 1, 1, 3)) / 2).astype(np.float32)
    wf = r.standard_normal((64, 3, 3, 1024)).astype(np.float32)
    a, b = (r.standard_normal(64) / 50).astype(np.float32), r.standard_normal(64).astype(np.float32)
    inits = [{"name": "w1", "shape": [1024, 1, 1, 3], "data": w1, "align_hwc_to_128": False},
             {"name": "w2", "shape": [64, 3, 3, 1024], "data": models.pack_weight(wf).ravel(), "align_hwc_to_128": True},
             {"name": "a", "shape": [64], "data": a, "align_hwc_to_128": False},
             {"name": "b", "shape": [64], "data": b, "align_hwc_to_128": False}]
    layers = [{"type": "FpConv2D", "name": "conv", "input": "data", "weight": "w1", "output": "wide", "pads": [0] * 4,
               "strides": [1, 1], "dilations": [1, 1]},
              {"type": "BinConv2D", "name": "bconv", "input": "wide", "weight": "w2", "output": "cnt", "pads": [1] * 4,
               "strides": [1, 1], "dilations": [1, 1]},
              {"type": "Affine", "name": "affine", "input": "cnt", "a": "a", "b": "b", "output": "cnt_bn"}]
    buf = df.write_model(layers, inits, [("data", [1, 9, 7, 3])])
    batch = 3
    x = r.standard_normal((batch, 9, 7, 3)).astype(np.float32)
    outs = []
    for optimize in (True, False):
        n = net.Net(batch=batch, optimize=optimize).read_buf(buf)
        descs = n.layers()
        assert sum(("DIRECT_CONV" if optimize else "BGEMM") in d for d in descs) == 1
        assert sum(d.startswith("Affine") for d in descs) == 1
        n.run(x)
        for i in range(batch):
            assert check_every_segment(n, layers, inits, i) == 2  # the in-place Affine belongs to the BinConv group
        outs.append(n.get_blob("cnt_bn").copy())
        n.close()
    np.testing.assert_array_equal(outs[0], outs[1])


def test_stem_fusion_leaves_other_graphs_alone(mods):
    """The convolution + MaxPool pass needs the pool to be the only reader of the convolution's blob and a 3x3 stride-2
    pad-1 window: a second reader, or another window, keeps both layers, and every blob stays readable."""
    df, models, net = mods
    r = np.random.default_rng(13)
    w = (r.standard_normal((64, 7, 7, 3)) / 12).astype(np.float32)
    inits = [{"name": "w", "shape": [64, 7, 7, 3], "data": w, "align_hwc_to_128": False}]
    conv = {"type": "FpConv2D", "name": "conv", "input": "data", "weight": "w", "output": "conv_out", "pads": [3] * 4,
            "strides": [2, 2], "dilations": [1, 1]}
    pool = {"type": "MaxPool", "name": "pool", "input": "conv_out", "output": "pool_out", "kernel_shape": [3, 3],
            "pads": [1] * 4, "strides": [2, 2]}
    other = {"type": "AvePool", "name": "avg", "input": "conv_out", "output": "avg_out", "kernel_shape": [2, 2],
             "pads": [0] * 4, "strides": [2, 2]}
    pool2 = dict(pool, kernel_shape=[2, 2], pads=[0] * 4)
    batch = 8
    x = r.standard_normal((batch, 224, 224, 3)).astype(np.float32)
    for layers, fused in (([conv, pool], True), ([conv, pool, other], False), ([conv, pool2], False)):
        n = net.Net(batch=batch).read_buf(df.write_model(layers, inits, [("data", [1, 224, 224, 3])]))
        descs = n.layers()
        assert any("+ MaxPool 3x3 stride 2" in d for d in descs) == fused, descs
        assert len(descs) == (len(layers) - 1 if fused else len(layers))
        n.run(x)
        gone = blobs_not_produced(n, layers)
        assert gone == ({"conv_out"} if fused else set())
        for i in (0, batch - 1):
            assert check_every_segment(n, layers, inits, i, gone) == len(layers) - len(gone)
        n.close()


def test_error_paths(mods, tmp_path):
    df, models, net = mods
    with pytest.raises(ValueError, match="Open file error"):  # std::invalid_argument, dabnn/net.cpp:34-36
        net.Net().read(str(tmp_path / "missing.dab"))
    layers, inits, inputs = models.small_bnn(0)
    with pytest.raises(RuntimeError, match="model version should be 2"):
        net.Net().read_buf(df.write_model(layers, inits, inputs, version=1))
    with pytest.raises(RuntimeError, match="fconv must be run in strict mode"):
        net.Net(run_fconv=False, strict=True).read_buf(df.write_model(layers, inits, inputs))
    bad = layers + [{"type": "Softmax", "name": "sm", "input": "logits", "output": "prob"}]
    with pytest.raises(RuntimeError, match="Not supported op Softmax"):
        net.Net().read_buf(df.write_model(bad, inits, inputs))
    shuffle = [{"type": "Shuffle", "name": "sh", "input": "data", "output": "out"}]
    with pytest.raises(RuntimeError, match="Shuffle only supports bit mat"):  # dabnn/layers/Shuffle.h:16-18
        net.Net().read_buf(df.write_model(shuffle, [], [("data", [1, 4, 4, 128])]))
    # a weight tensor shorter than the layer's geometry is refused before any kernel could read past it
    wp = models.pack_weight(np.ones((8, 3, 3, 128), np.float32))
    short = [{"name": "w", "shape": [8, 3, 3, 128], "data": np.ascontiguousarray(wp[:, :16]).ravel(), "align_hwc_to_128": True}]
    conv = [{"type": "BinConv2D", "name": "bc", "input": "data", "weight": "w", "output": "cnt", "pads": [1] * 4,
             "strides": [1, 1], "dilations": [1, 1]}]
    with pytest.raises(RuntimeError, match="words per filter"):
        net.Net().read_buf(df.write_model(conv, short, [("data", [1, 8, 8, 128])]))
    good = df.write_model(layers, inits, inputs)
    with pytest.raises(ValueError, match="malformed model buffer"):  # std::invalid_argument
        net.Net().read_buf(good[:len(good) // 2])
    n = net.Net().read_buf(df.write_model(layers, inits, inputs))
    with pytest.raises(KeyError):
        n.get_blob("no_such_blob")
    with pytest.raises(ValueError):
        n.run(np.zeros((1, 8, 8, 3), dtype=np.float32))
    n.close()


def test_split_and_shuffle_layers_on_bit_blobs(mods):
    """dabnn/net.cpp:245-256: Shuffle works in place on a Bit blob, Split cuts it into two Bit blobs.  No layer of
    the reference's Net produces a Bit blob, so the input is a Bit initializer, as in the reference."""
    df, models, net = mods
    r = np.random.default_rng(15)
    for c in (128, 256, 384, 512):
        words = r.integers(0, 2**64, size=(3, 5, 4, c // 64), dtype=np.uint64)
        inits = [{"name": "bits", "shape": [3, 5, 4, c], "data": words.ravel(), "align_hwc_to_128": False}]
        layers = [{"type": "Shuffle", "name": "sh", "input": "bits", "output": "shuffled"},
                  {"type": "Split", "name": "sp", "input": "shuffled", "outputs": ["left", "right"]}]
        n = net.Net(batch=2).read_buf(df.write_model(layers, inits, [("data", [1, 4, 4, 64])]))
        assert [d.split()[0] for d in n.layers()] == ["Shuffle", "Split"]
        n.run(np.zeros((2, 4, 4, 64), np.float32))
        want = orc.shuffle_bit(words.copy())
        l, rgt = orc.split_bit(want)
        np.testing.assert_array_equal(n.get_blob("shuffled").reshape(want.shape), want)
        np.testing.assert_array_equal(n.get_blob("bits").reshape(want.shape), want)  # in place: the names alias
        np.testing.assert_array_equal(n.get_blob("left").reshape(l.shape), l)
        np.testing.assert_array_equal(n.get_blob("right").reshape(rgt.shape), rgt)
        n.close()


def test_flatc_style_encoding_loads(mods):
    """Files written the way flatc's builders write them -- default scalars left out (Float32 tensors, the FpConv2D
    layer type, align_hwc_to_128 = false), equal vtables shared, trailing absent slots trimmed from every vtable,
    four-entry symmetric pads -- give the same network as the untrimmed encoding."""
    df, models, net = mods
    layers, inits, inputs = models.small_bnn(5, hw=16, width=64)
    assert any(len(l.get("pads", [])) == 4 for l in layers)
    plain = df.write_model(layers, inits, inputs)
    trimmed = df.write_model(layers, inits, inputs, trim_vtables=True)
    assert len(trimmed) < len(plain)
    x = np.random.default_rng(16).standard_normal((2, 16, 16, 3)).astype(np.float32)
    outs = []
    for buf in (plain, trimmed):
        n = net.Net(batch=2).read_buf(buf)
        outs.append(n.layers())
        n.run(x)
        outs.append(n.get_blob("logits").copy())
        n.close()
    assert outs[0] == outs[2]
    np.testing.assert_array_equal(outs[1], outs[3])


def test_cpp_callers_of_the_reference_work_unchanged(mods, tmp_path):
    """tests/cpp/net_api_test.cpp is the reference's own usage (tests/net_test.cpp:29-50,63-65, JavaWrapper.cpp:56-60,
    binaries/run.cpp:41-50) compiled against this library's C++ headers: optimize = false and optimize = true agree
    through Mat::operator==, and get_blob hands back host-readable data through data, operator T*, operator[]."""
    import os
    import subprocess
    df, models, net = mods
    exe = os.path.join(os.path.dirname(os.path.abspath(net.__file__)), "lib", "net_api_test")
    assert os.path.exists(exe), "build it with make -C dabnn_amd/host"
    layers, inits, inputs = models.small_bnn(6, hw=16, width=64)
    path = tmp_path / "small.dab"
    path.write_bytes(df.write_model(layers, inits, inputs))
    out = subprocess.run([exe, str(path), "logits", str(16 * 16 * 3), "binaized_for_b0_cnt_cal"], capture_output=True,
                         text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.strip().endswith("ok")
    n = net.Net(batch=1).read_buf(path.read_bytes())
    n.run(np.ones((1, 16, 16, 3), np.float32))
    want = n.get_blob("logits").ravel()
    got = [float(l.split()[2]) for l in out.stdout.splitlines() if l.startswith("v ")]
    assert len(got) == 8
    np.testing.assert_array_equal(np.array(got, np.float32), want[:8])
    w0 = [int(l.split()[1]) for l in out.stdout.splitlines() if l.startswith("w0 ")]
    assert w0 == [int(n.get_blob("binaized_for_b0_cnt_cal").ravel()[0])]
    n.close()


def test_graph_replay_equals_eager(mods):
    """Runs 3+ replay a captured HIP graph; every replay must equal the eager result, also with other GPU work
    and synchronisations in between and with changing inputs."""
    import torch
    df, models, net = mods
    layers, inits, inputs = models.small_bnn(4, hw=16, width=64)
    buf = df.write_model(layers, inits, inputs)
    r = np.random.default_rng(9)
    xs = [r.standard_normal((2, 16, 16, 3)).astype(np.float32) for _ in range(6)]
    eager = net.Net(batch=2).read_buf(buf)
    eager.set_use_graph(False)
    graphed = net.Net(batch=2).read_buf(buf)
    for i, x in enumerate(xs):
        eager.run(x)
        want = eager.get_blob("logits").copy()
        graphed.run(x)  # runs 0 and 1 eager, run 2 captures, later runs replay
        got = graphed.get_blob("logits").copy()
        np.testing.assert_array_equal(got, want, err_msg="run %d" % i)
        torch.randn(1 << 16, device="cuda").sum().item()  # unrelated eager work and a sync between replays
    eager.close()
    graphed.close()


def test_run_device_reads_the_callers_buffer_in_place(mods):
    """A device input is read where it lies (the reference's run wraps its pointer without a copy): the same buffer
    run after run replays the captured graph and sees new contents, another buffer makes the net capture again, from
    the third change on the net copies into its own blob, and an unaligned buffer is copied from the start.  Every
    run gives the logits of the same input passed from the host."""
    import torch
    df, models, net = mods
    layers, inits, inputs = models.small_bnn(6, hw=16, width=64)
    buf = df.write_model(layers, inits, inputs)
    r = np.random.default_rng(17)
    batch = 3
    xs = [r.standard_normal((batch, 16, 16, 3)).astype(np.float32) for _ in range(12)]
    ref = net.Net(batch=batch).read_buf(buf)
    ref.set_use_graph(False)
    want = [ref.run(x).get_blob("logits").copy() for x in xs]
    ref.close()

    n = net.Net(batch=batch).read_buf(buf)
    a = torch.empty((batch, 16, 16, 3), device="cuda")
    keep = a.clone()
    for i in range(5):  # one buffer, new contents every run: two eager runs, the capture, two replays
        a.copy_(torch.from_numpy(xs[i]))
        keep.copy_(a)
        np.testing.assert_array_equal(n.run(a).get_blob("logits"), want[i], err_msg="run %d" % i)
        assert torch.equal(a, keep), "the net wrote into the caller's buffer"
        np.testing.assert_array_equal(n.get_blob(n.input_name), xs[i])
    others = [torch.from_numpy(xs[i]).cuda() for i in range(5, 10)]  # a new buffer every run
    for i, t in zip(range(5, 10), others):
        np.testing.assert_array_equal(n.run(t).get_blob("logits"), want[i], err_msg="run %d" % i)
        np.testing.assert_array_equal(n.get_blob(n.input_name), xs[i])
    np.testing.assert_array_equal(n.run(xs[10]).get_blob("logits"), want[10])  # a host input in between
    flat = torch.empty(batch * 16 * 16 * 3 + 8, device="cuda")
    odd = flat[1:1 + batch * 16 * 16 * 3].view(batch, 16, 16, 3)  # four bytes off the allocation's alignment
    assert odd.data_ptr() % 256 != 0 and odd.is_contiguous()
    odd.copy_(torch.from_numpy(xs[11]))
    np.testing.assert_array_equal(n.run(odd).get_blob("logits"), want[11])
    np.testing.assert_array_equal(n.run(a).get_blob("logits"), want[4])
    n.close()

    # a fresh net, an unaligned buffer from the first run on and through the capture
    m = net.Net(batch=batch).read_buf(buf)
    for i in range(4):
        odd.copy_(torch.from_numpy(xs[i]))
        np.testing.assert_array_equal(m.run(odd).get_blob("logits"), want[i], err_msg="run %d" % i)
    m.close()


def test_run_device_copies_when_a_layer_rewrites_the_input_blob(mods):
    """An in-place layer on the input blob (an Affine that normalises the image) must not write into the caller's
    device buffer: such a net copies its input."""
    import torch
    df, models, net = mods
    r = np.random.default_rng(19)
    a, b = r.standard_normal(4).astype(np.float32), r.standard_normal(4).astype(np.float32)
    w = (r.standard_normal((8, 3, 3, 4)) / 6).astype(np.float32)
    inits = [{"name": "a", "shape": [4], "data": a, "align_hwc_to_128": False},
             {"name": "b", "shape": [4], "data": b, "align_hwc_to_128": False},
             {"name": "w", "shape": [8, 3, 3, 4], "data": w, "align_hwc_to_128": False}]
    layers = [{"type": "Affine", "name": "norm", "input": "data", "a": "a", "b": "b", "output": "data_n"},
              {"type": "FpConv2D", "name": "conv", "input": "data_n", "weight": "w", "output": "conv_out", "pads": [1] * 4,
               "strides": [1, 1], "dilations": [1, 1]}]
    n = net.Net(batch=2).read_buf(df.write_model(layers, inits, [("data", [1, 9, 9, 4])]))
    x = r.standard_normal((2, 9, 9, 4)).astype(np.float32)
    t = torch.from_numpy(x).cuda()
    for _ in range(4):
        got = n.run(t).get_blob("conv_out")
        assert torch.equal(t.cpu(), torch.from_numpy(x)), "the net wrote into the caller's buffer"
        for i in range(2):
            close(got[i], orc.fconv(orc.affine_inplace(x[i].copy(), a, b), w, None, 3, 3, 1, 1, 1, 1))
    n.close()


def test_nets_on_threads_of_their_own_do_not_disturb_each_other(mods):
    """Every Net has a stream of its own: nets that are read, run (eager runs, the capture of the HIP graph on the
    third run, replays), read back and destroyed on two host threads at once give the logits each gives alone."""
    import threading
    df, models, net = mods
    layers, inits, inputs = models.bireal18(21, stem=False)
    buf = df.write_model(layers, inits, inputs)
    r = np.random.default_rng(13)
    batches = (3, 8)
    xs = [[r.standard_normal((b, 224, 224, 3)).astype(np.float32) for _ in range(5)] for b in batches]
    alone = []
    for b, inputs_ in zip(batches, xs):
        ref = net.Net(batch=b).read_buf(buf)
        ref.set_use_graph(False)
        alone.append([ref.run(x).get_blob("logits").copy() for x in inputs_])
        ref.close()
    rounds = 4
    got = [[], []]
    errors = []
    start = threading.Barrier(2)

    def work(i):
        try:
            start.wait()
            for _ in range(rounds):
                n = net.Net(batch=batches[i]).read_buf(buf)
                got[i].append([n.run(x).get_blob("logits").copy() for x in xs[i]])
                n.close()
        except Exception as e:  # noqa: BLE001 - reported by the assertion below
            errors.append("thread %d: %r" % (i, e))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        assert len(got[i]) == rounds
        for k, one_round in enumerate(got[i]):
            for j, (g, w) in enumerate(zip(one_round, alone[i])):
                np.testing.assert_array_equal(g, w, err_msg="thread %d round %d run %d" % (i, k, j))
