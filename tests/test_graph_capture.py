"""Launches of the library recorded into a HIP graph (mi355_graph_*) and
replayed: a decode matmul in the packed int4 layout, a small int8 GEMM, a
bf16 GEMM with a layout copy in its launch, a grouped matmul on the tiles and a
reorder, all in one graph.  Every replay must reproduce the eager results bit
for bit; between replays the dst buffers are overwritten from the host and
the program synchronizes, so a replay that does nothing, or only works the
first time, shows."""
import ctypes as C

import numpy as np
import pytest

from onednn_amd import cabi, configs
from tests import grouped_cases as gc


def decode_problem(M):
    p = configs.config2(M=M, N=512, K=1024, wtag="ab")
    p.wei_packing = cabi.WEI_PACK_WOQ64
    return p


class GroupedRun:
    def __init__(self, p, stream):
        from onednn_amd.grouped import fill_args
        self.lib, self.p, self.stream = cabi.load_kernels(), p, stream
        self.d = p.desc()
        self.bufs = []

        def place(arr):
            b = cabi.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))
            self.bufs.append(b)
            return b.ptr

        self.a = fill_args(p, place)
        self.init = p.initial_dst()
        self.dst = cabi.DeviceBuffer.from_numpy(self.init)
        self.a.dst = self.dst.ptr

    def launch(self):
        cabi.check(self.lib.mi355_grouped_matmul_launch(C.byref(self.d), C.byref(self.a), self.stream))

    def reset_dst(self):
        self.dst.upload(self.init)

    def result(self):
        return self.dst.to_numpy(np.uint8, self.init.shape)

    def free(self):
        for b in self.bufs + [self.dst]:
            b.free()


@pytest.mark.gpu
def test_a_graph_of_launches_replays_the_eager_results(gpu):
    from onednn_amd.problem import GpuRun
    from onednn_amd.reorder import GpuReorder, ReorderProblem
    stream = cabi.Stream()
    runs = [GpuRun(decode_problem(1), stream=stream.ptr), GpuRun(decode_problem(32), stream=stream.ptr),
            GpuRun(configs.config1(wtag="ba"), stream=stream.ptr),
            GpuRun(configs.config_h16(M=256, N=384, K=320, wtag="ab"), stream=stream.ptr)]
    gp, _ = gc.case_2dx3d([5, 0, 17, 9], 128, 64, src_dt=cabi.DT_F8_E4M3, wei_dt=cabi.DT_F8_E4M3, dst_dt=cabi.DT_BF16,
                          wtag="acb", src_scale="row", wei_scale="col")
    runs.append(GroupedRun(gp, stream.ptr))
    impls = [cabi.impl_name(r.impl) for r in runs[:4]]
    assert impls[0].startswith("hip:woq_packed") and impls[1].startswith("hip:woq_packed"), impls
    assert impls[2].startswith("hip:mfma_i8") and impls[3].startswith("hip:mfma_h16"), impls

    # eager: the results to reproduce (and whatever a first launch sets up happens here, outside the capture)
    for r in runs:
        r.launch()
    stream.sync()
    want = [np.array(r.result(), copy=True) for r in runs]

    with cabi.Graph(stream) as g:
        for r in runs:
            r.launch()
        for r in runs[:2]:      # a kernel recorded twice
            r.launch()
    try:
        for replay in range(3):
            for r in runs:
                r.reset_dst()
            stream.sync()
            for r, w in zip(runs, want):       # nothing ran while recording, and the reset took
                if replay == 0:
                    assert not np.array_equal(r.result(), w)
            g.launch()
            stream.sync()
            for i, (r, w) in enumerate(zip(runs, want)):
                assert np.array_equal(r.result(), w), f"replay {replay}, launch {i}"
    finally:
        g.destroy()
        for r in runs:
            r.free()
        stream.destroy()


@pytest.mark.gpu
def test_capture_needs_a_created_stream(gpu):
    lib = cabi.load_kernels()
    assert lib.mi355_graph_capture_begin(None) == cabi.INVALID_ARGUMENTS
    assert lib.mi355_graph_launch(None, None) == cabi.INVALID_ARGUMENTS
    assert lib.mi355_graph_destroy(None) == cabi.SUCCESS


@pytest.mark.gpu
def test_a_primitive_on_the_callers_stream_is_ordered_and_captured_with_it(gpu):
    """dnnl_amd_interop_stream_create: the dnnl stream is the caller's hipStream_t.  A fill enqueued on that stream by
    the caller, then the primitive through the dnnl layer, no host synchronization between them; then the execute
    call recorded into the caller's graph and replayed."""
    from onednn_amd import dnnl
    from tests.test_gpu_dnnl_api import run_through_api
    lib = cabi.load_kernels()
    p = configs.config3(M=256, N=256, K=512)
    want, impl, (pd, prim, strm0, args) = run_through_api(p)      # eager, on a stream of the library's
    assert impl.startswith("hip:mfma_i8")
    hs = cabi.Stream()
    strm = dnnl.stream(strm0.engine, hip_stream=hs.ptr)
    assert strm.hip_stream() == hs.ptr
    dst = args[dnnl.ARG_DST]
    handle = dst.get_data_handle()
    try:
        cabi.check(lib.mi355_mem_set(handle, 0x55, dst.md.get_size(), hs.ptr))
        prim.execute(strm, args)
        strm.wait()
        assert np.array_equal(dst.read(np.int8), want)

        with cabi.Graph(hs) as g:
            prim.execute(strm, args)
        for _ in range(2):
            dst.write(np.full(want.shape, 0x33, np.int8))
            assert not np.array_equal(dst.read(np.int8), want)
            g.launch()
            hs.sync()
            assert np.array_equal(dst.read(np.int8), want)
        g.destroy()
    finally:
        hs.destroy()
