"""HIP graph capture of C-ABI calls: every entry point of the hot path issues nothing but kernel launches on the
context's stream, so a caller may record them into a graph.  The graph is replayed several times with new operand
contents, eager calls and synchronisations in between, and every replay is compared with the eager result on the
same operands (bit for bit: the operators here are integer ones)."""
import numpy as np
import pytest

from reference_model_amd import Context, capi

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def test_graph_of_the_int8_layer_chain_matches_eager_on_every_replay():
    dev = torch.device("cuda:0")
    ctx = Context(0)
    try:
        stream = torch.cuda.current_stream()
        ctx.set_stream(stream.cuda_stream)
        rng = np.random.default_rng(8)
        n, hw, c = 4, 28, 64
        x = torch.empty((n, hw, hw, c), dtype=torch.int8, device=dev)
        w = torch.from_numpy(rng.integers(-127, 128, (c, 3, 3, c)).astype(np.int8)).to(dev)
        bias = torch.from_numpy(rng.integers(-9999, 9999, c).astype(np.int32)).to(dev)
        mult = torch.from_numpy(rng.integers(1 << 30, 1 << 31, c).astype(np.int32)).to(dev)
        shift = torch.from_numpy(rng.integers(38, 42, c).astype(np.int8)).to(dev)
        wd = torch.from_numpy(rng.integers(-127, 128, (3, 3, c, 1)).astype(np.int8)).to(dev)
        y = torch.empty((n, hw, hw, c), dtype=torch.int8, device=dev)      # CONV2D + RESCALE + CLAMP
        z = torch.empty((n, hw, hw, c), dtype=torch.int8, device=dev)      # DEPTHWISE_CONV2D + RESCALE
        p = torch.empty((n, hw // 2, hw // 2, c), dtype=torch.int8, device=dev)    # MAX_POOL2D
        rows = (hw // 2) * (hw // 2)
        m = torch.empty((n, rows, hw // 2), dtype=torch.int32, device=dev)         # MATMUL [n, rows, c] x [n, c, hw/2]
        pt = torch.empty((n, c, hw // 2), dtype=torch.int8, device=dev)
        d = ctx.conv_desc(capi.INT8, capi.INT32, (n, hw, hw, c), c, 3, 3, (hw, hw), (1, 1, 1, 1), (1, 1), (1, 1), c)
        r = ctx.rescale_desc(capi.INT32, capi.INT8, c, c, 0, -3, True, capi.ROUND_DOUBLE, True, False, False)
        pd = capi.PoolDesc()
        pd.dtype, pd.N, pd.IH, pd.IW, pd.C, pd.OH, pd.OW = capi.INT8, n, hw, hw, c, hw // 2, hw // 2
        pd.kernel[:], pd.stride[:], pd.pad[:] = [2, 2], [2, 2], [0, 0, 0, 0]
        pd.nan_mode, pd.acc_dtype = 1, capi.INT32

        def chain():
            ctx.conv2d_rescale_clamp(d, x, w, bias, -7, 0, r, mult, shift, y, (-100, 100))
            ctx.depthwise_conv2d_rescale_clamp(d, y, wd, bias, 5, 0, r, mult, shift, z, None)
            ctx.max_pool2d(pd, z, p)
            ctx.matmul(capi.INT8, n, rows, c, hw // 2, p, pt, 2, -1, m)

        def fresh_inputs(seed):
            g = np.random.default_rng(seed)
            x.copy_(torch.from_numpy(g.integers(-128, 128, tuple(x.shape)).astype(np.int8)))
            pt.copy_(torch.from_numpy(g.integers(-128, 128, tuple(pt.shape)).astype(np.int8)))

        fresh_inputs(0)
        chain()     # first calls outside the capture: one-time kernel attribute set-up happens here
        assert ctx.sync() == capi.VALID
        kernels = ctx.last_kernel
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.graph(graph, stream=side):
            ctx.set_stream(side.cuda_stream)
            chain()
        ctx.set_stream(stream.cuda_stream)
        for seed in (1, 2, 3, 4):
            fresh_inputs(seed)
            chain()                                    # eager, on the same operands
            assert ctx.sync() == capi.VALID
            want = [t.clone() for t in (y, z, p, m)]
            for t in (y, z, p, m):
                t.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert ctx.sync() == capi.VALID
            for got, ref in zip((y, z, p, m), want):
                assert torch.equal(got, ref)
            assert len(torch.unique(y)) > 50 and len(torch.unique(m)) > 50
        assert kernels.startswith("matmul")
    finally:
        ctx.close()


def test_graph_of_transpose_conv_conv3d_and_avg_pool_matches_eager_on_every_replay():
    """TRANSPOSE_CONV2D and CONV3D once through the kernel that reads their operands in place (one launch, no scratch
    buffer) and once through the re-laid-out operands (scratch buffer grown by the eager pass before the capture),
    and AVG_POOL2D."""
    dev = torch.device("cuda:0")
    ctx = Context(0)
    try:
        stream = torch.cuda.current_stream()
        ctx.set_stream(stream.cuda_stream)
        rng = np.random.default_rng(21)
        n, hw, c, oc = 2, 12, 64, 64
        x = torch.empty((n, hw, hw, c), dtype=torch.int8, device=dev)
        wt = torch.from_numpy(rng.integers(-127, 128, (oc, 3, 3, c)).astype(np.int8)).to(dev)
        bias = torch.from_numpy(rng.integers(-9999, 9999, oc).astype(np.int32)).to(dev)
        up = 2 * (hw - 1) + 3
        t_out = torch.empty((n, up, up, oc), dtype=torch.int32, device=dev)
        t_out2 = torch.empty_like(t_out)
        td = capi.TconvDesc()
        td.in_dtype, td.out_dtype = capi.INT8, capi.INT32
        td.N, td.IH, td.IW, td.IC, td.OC, td.KH, td.KW, td.OH, td.OW = n, hw, hw, c, oc, 3, 3, up, up
        td.out_pad[:], td.stride[:], td.bias_len = [0, 0, 0, 0], [2, 2], oc
        v = torch.empty((1, 6, 10, 10, 32), dtype=torch.int8, device=dev)
        w3 = torch.from_numpy(rng.integers(-127, 128, (oc, 3, 3, 3, 32)).astype(np.int8)).to(dev)
        c_out = torch.empty((1, 6, 10, 10, oc), dtype=torch.int32, device=dev)
        c_out2 = torch.empty_like(c_out)
        cd = capi.Conv3dDesc()
        cd.in_dtype, cd.out_dtype = capi.INT8, capi.INT32
        cd.N, cd.ID, cd.IH, cd.IW, cd.IC, cd.OC, cd.KD, cd.KH, cd.KW, cd.OD, cd.OH, cd.OW = 1, 6, 10, 10, 32, oc, 3, 3, 3, 6, 10, 10
        cd.pad[:], cd.stride[:], cd.dilation[:], cd.bias_len = [1] * 6, [1] * 3, [1] * 3, oc
        pd = capi.PoolDesc()
        pd.dtype, pd.N, pd.IH, pd.IW, pd.C, pd.OH, pd.OW = capi.INT8, n, hw, hw, c, hw // 2, hw // 2
        pd.kernel[:], pd.stride[:], pd.pad[:] = [2, 2], [2, 2], [0, 0, 0, 0]
        pd.nan_mode, pd.acc_dtype = 1, capi.INT32
        p_out = torch.empty((n, hw // 2, hw // 2, c), dtype=torch.int8, device=dev)
        names = []

        def chain():
            ctx.set_kernel_choice(capi.KERNEL_AUTO)
            ctx.transpose_conv2d(td, x, wt, bias, -5, 0, t_out)
            names.append(ctx.last_kernel)
            ctx.conv3d(cd, v, w3, bias, 3, 0, c_out)
            names.append(ctx.last_kernel)
            ctx.set_kernel_choice(capi.KERNEL_MFMA)
            ctx.transpose_conv2d(td, x, wt, bias, -5, 0, t_out2)
            ctx.conv3d(cd, v, w3, bias, 3, 0, c_out2)
            ctx.set_kernel_choice(capi.KERNEL_AUTO)
            ctx.avg_pool2d(pd, x, -5, 7, p_out)

        def fresh_inputs(seed):
            g = np.random.default_rng(seed)
            x.copy_(torch.from_numpy(g.integers(-128, 128, tuple(x.shape)).astype(np.int8)))
            v.copy_(torch.from_numpy(g.integers(-128, 128, tuple(v.shape)).astype(np.int8)))

        fresh_inputs(0)
        chain()     # the eager pass sets kernel attributes and grows the scratch buffer
        assert ctx.sync() == capi.VALID
        assert names[:2] == ["transpose_conv2d_slab_i8", "conv3d_slab_i8"]
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.graph(graph, stream=side):
            ctx.set_stream(side.cuda_stream)
            chain()
        ctx.set_stream(stream.cuda_stream)
        outs = (t_out, t_out2, c_out, c_out2, p_out)
        for seed in (1, 2, 3):
            fresh_inputs(seed)
            chain()
            assert ctx.sync() == capi.VALID
            want = [t.clone() for t in outs]
            assert torch.equal(want[0], want[1]) and torch.equal(want[2], want[3])
            for t in outs:
                t.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert ctx.sync() == capi.VALID
            for got, ref in zip(outs, want):
                assert torch.equal(got, ref)
            assert len(torch.unique(t_out)) > 50 and len(torch.unique(c_out)) > 50 and len(torch.unique(p_out)) > 20
    finally:
        ctx.close()
