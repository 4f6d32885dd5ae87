"""The steady-state calls enqueue kernels only (no allocation, no memset, no synchronisation), so a
caller may capture them into a HIP graph and replay it: SpMV (vector and merge family, once the
plan of the matrix is cached), SpMM with and without a schedule, csr2csc.  Every replay is checked
against the CPU oracle, with eager work and synchronisations in between and new operand values
each time.

Reference: the calls are plain stream work there too (mcsp_spmv_gpu.cpp:203-259 launches on
handle->stream); the reference's SpMM synchronises and allocates (mcsp_spmm_gpu.cpp:119-160) and
could not be captured."""
import numpy as np
import pytest

from mcsparse_amd import api
from mcsparse_amd import workloads as wl

from gpu_util import assert_within, dev

pytestmark = pytest.mark.gpu


def test_calls_replay_in_a_hip_graph(torch_gpu, oracle):
    torch = torch_gpu
    rng = np.random.default_rng(21)
    side = torch.cuda.Stream()
    handle = api.Handle(stream=side.cuda_stream)

    a = wl.random_ragged(4000, 3000, 12, dtype=np.float64, seed=7)               # vector family
    p = wl.power_law(m=6000, max_len=5000, dtype=np.float32)                     # merge family
    s = wl.stencil_27pt(12, dtype=np.float32)                                    # SpMM, csr2csc
    n_cols = 24

    def upload(mat):
        return dev(torch, mat.ptr), dev(torch, mat.col), dev(torch, mat.val)

    held = []  # device arrays the descriptors point at
    d_a, d_p, d_s = upload(a), upload(p), upload(s)
    held += [d_a, d_p, d_s]
    A = api.SpMat(a.m, a.n, a.nnz, *d_a, base=a.base)
    A.set_plan(api.FAMILY_VECTOR)  # both families take part in the graph: this one by request, P by analysis
    P = api.SpMat(p.m, p.n, p.nnz, *d_p, base=p.base)
    S = api.SpMat(s.m, s.n, s.nnz, *d_s, base=s.base)

    x_a = torch.zeros(a.n, dtype=torch.float64, device="cuda")
    y_a = torch.zeros(a.m, dtype=torch.float64, device="cuda")
    x_p = torch.zeros(p.n, dtype=torch.float32, device="cuda")
    y_p = torch.zeros(p.m, dtype=torch.float32, device="cuda")
    B = torch.zeros(s.n, n_cols, dtype=torch.float32, device="cuda")
    C = torch.zeros(s.m, n_cols, dtype=torch.float32, device="cuda")
    C2 = torch.zeros(s.m, n_cols, dtype=torch.float32, device="cuda")
    t_val = torch.zeros(s.nnz, dtype=torch.float32, device="cuda")
    t_ptr = torch.zeros(s.n + 1, dtype=torch.int32, device="cuda")
    t_row = torch.zeros(s.nnz, dtype=torch.int32, device="cuda")

    vx_a, vy_a, vx_p, vy_p = api.DnVec(x_a), api.DnVec(y_a), api.DnVec(x_p), api.DnVec(y_p)
    mB, mC, mC2 = api.DnMat(s.n, n_cols, n_cols, B), api.DnMat(s.m, n_cols, n_cols, C), api.DnMat(s.m, n_cols, n_cols, C2)

    def scratch(status_and_size):
        st, size = status_and_size
        assert st == 0
        return torch.empty(size, dtype=torch.uint8, device="cuda")

    buf_a = scratch(api.spmv_buffer_size(handle, api.OP_N, 1.5, A, vx_a, 0.0, vy_a, api.R_64F))
    buf_p = scratch(api.spmv_buffer_size(handle, api.OP_N, 1.0, P, vx_p, 0.0, vy_p, api.R_32F))
    buf_s = scratch(api.spmm_buffer_size(handle, 0, 0, 2.0, S, mB, 0.0, mC, api.R_32F))
    buf_s2 = scratch(api.spmm_buffer_size(handle, 0, 0, 2.0, S, mB, 0.0, mC2, api.R_32F))
    buf_t = scratch(api.csr2csc_buffer_size(handle, s.m, s.n, s.nnz, d_s[2], d_s[0], d_s[1], t_val, t_ptr, t_row,
                                            api.R_32F, api.ACTION_NUMERIC, s.base))

    def enqueue():
        assert api.spmv(handle, api.OP_N, 1.5, A, vx_a, 0.0, vy_a, api.R_64F, buf_a) == 0
        assert api.spmv(handle, api.OP_N, 1.0, P, vx_p, 0.0, vy_p, api.R_32F, buf_p) == 0
        assert api.spmm(handle, 0, 0, 2.0, S, mB, 0.0, mC, api.R_32F, buf_s) == 0      # scheduled
        assert api.spmm(handle, 0, 0, 2.0, S, mB, 0.0, mC2, api.R_32F, buf_s2) == 0    # schedule-free
        assert api.csr2csc(handle, s.m, s.n, s.nnz, d_s[2], d_s[0], d_s[1], t_val, t_ptr, t_row, api.R_32F,
                           api.ACTION_NUMERIC, s.base, buf_t) == 0

    with torch.cuda.stream(side):
        # the first SpMV on a structure reads its row statistics back and the schedule build reads two
        # counters back: both block, so they happen before the capture
        assert api.spmm_preprocess(handle, 0, 0, 2.0, S, mB, 0.0, mC, api.R_32F, buf_s) == 0
        enqueue()
    torch.cuda.synchronize()
    assert A.plan()[0] == api.FAMILY_VECTOR and P.plan()[0] == api.FAMILY_MERGE

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue()
    torch.cuda.synchronize()

    want_t = oracle.csr2csc(s.m, s.n, s.base, s.ptr, s.col, s.val, method="counting")
    for replay in range(3):
        hx_a = rng.uniform(-1, 1, a.n)
        hx_p = rng.uniform(-1, 1, p.n).astype(np.float32)
        hB = rng.uniform(-1, 1, (s.n, n_cols)).astype(np.float32)
        x_a.copy_(torch.from_numpy(hx_a))
        x_p.copy_(torch.from_numpy(hx_p))
        B.copy_(torch.from_numpy(hB))
        for out in (y_a, y_p, C, C2, t_val, t_ptr, t_row):
            out.fill_(-3)  # eager work between the replays; the graph must write every output again
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()

        ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.5, 0.0, hx_a, np.zeros(a.m))
        assert_within(y_a.cpu().numpy(), ref, bound, np.float64, what="replay %d, vector SpMV" % replay)
        ref, bound = oracle.spmv(False, p.m, p.n, p.base, p.ptr, p.col, p.val, 1.0, 0.0, hx_p,
                                 np.zeros(p.m, np.float32))
        assert_within(y_p.cpu().numpy(), ref, bound, np.float32, what="replay %d, merge SpMV" % replay)
        ref, bound = oracle.spmm(s.m, n_cols, s.base, s.ptr, s.col, s.val, 2.0, 0.0, hB.ravel(), n_cols, True,
                                 np.zeros(s.m * n_cols, np.float32), n_cols, True)
        assert_within(C.cpu().numpy(), ref, bound, np.float32, what="replay %d, scheduled SpMM" % replay)
        assert_within(C2.cpu().numpy(), ref, bound, np.float32, what="replay %d, SpMM" % replay)
        assert np.array_equal(t_ptr.cpu().numpy().view(np.uint32), want_t[0])
        assert np.array_equal(t_row.cpu().numpy().view(np.uint32), want_t[1])
        assert np.array_equal(t_val.cpu().numpy().view(np.uint8), want_t[2].view(np.uint8))
    del graph
    torch.cuda.synchronize()
    handle.destroy()


@pytest.mark.parametrize("alg,state,tall", [(api.SPMV_ALG_DEFAULT, 3, False), (api.SPMV_CSR_ALG2, 2, False),
                                            (api.SPMV_ALG_DEFAULT, 3, True)])
def test_preprocessed_spmv_replays_in_a_hip_graph(torch_gpu, oracle, alg, state, tall):
    """mcsparseSpMV on a copy built by mcsparseSpMV_preprocess (before the capture: it blocks) is two kernels; one
    (which also puts its work counters back for the next replay) where x lies inside one band group (tall)."""
    torch = torch_gpu
    rng = np.random.default_rng(22)
    side = torch.cuda.Stream()
    handle = api.Handle(stream=side.cuda_stream)
    handle.set_spmv_preprocess_trial(False)  # the copy is what is replayed, whether or not it is the faster here
    a = wl.random_ragged(600000, 100000, 4, dtype=np.float64, seed=9) if tall else \
        wl.random_ragged(20000, 40000, 10, dtype=np.float64, seed=9)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    A = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    if not tall:
        A.set_band_bytes(1 << 13)
    x = torch.zeros(a.n, dtype=torch.float64, device="cuda")
    y = torch.zeros(a.m, dtype=torch.float64, device="cuda")
    vx, vy = api.DnVec(x), api.DnVec(y)
    st, size = api.spmv_preprocess_buffer_size(handle, api.OP_N, 1.5, A, vx, 0.5, vy, api.R_64F, alg=alg)
    assert st == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    with torch.cuda.stream(side):
        assert api.spmv_preprocess(handle, api.OP_N, 1.5, A, vx, 0.5, vy, api.R_64F, buf, alg=alg) == 0
        assert api.spmv(handle, api.OP_N, 1.5, A, vx, 0.5, vy, api.R_64F, buf, alg=alg) == 0
    torch.cuda.synchronize()
    assert A.spmv_preprocess_state()[0] == state
    assert not tall or A.spmv_preprocess_state()[1] == 1
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        # a preprocess call would have to block: refused on a capturing stream, the copy stays as it is
        assert api.spmv(handle, api.OP_N, 1.5, A, vx, 0.5, vy, api.R_64F, buf, alg=alg) == 0
    torch.cuda.synchronize()
    for replay in range(3):
        hx = rng.uniform(-1, 1, a.n)
        hy = rng.uniform(-1, 1, a.m)
        x.copy_(torch.from_numpy(hx))
        y.copy_(torch.from_numpy(hy))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 1.5, 0.5, hx, hy)
        assert_within(y.cpu().numpy(), ref, bound, np.float64, what="replay %d, state %d" % (replay, state))
    del graph
    torch.cuda.synchronize()
    handle.destroy()


@pytest.mark.parametrize("alg", [api.SPMV_ALG_DEFAULT, api.SPMV_CSR_ALG2])
def test_transposing_spmv_replays_in_a_hip_graph(torch_gpu, oracle, alg):
    """op T without a preprocess call: the sort passes and the column sums (in LDS by default, in row order under
    MCSPARSE_SPMV_CSR_ALG2) are kernels only, whatever the algorithm."""
    torch = torch_gpu
    rng = np.random.default_rng(23)
    side = torch.cuda.Stream()
    handle = api.Handle(stream=side.cuda_stream)
    a = wl.random_ragged(9000, 70001, 14, dtype=np.float32, seed=10, base=1)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    A = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    x = torch.zeros(a.m, dtype=torch.float32, device="cuda")
    y = torch.zeros(a.n, dtype=torch.float32, device="cuda")
    vx, vy = api.DnVec(x), api.DnVec(y)
    st, size = api.spmv_buffer_size(handle, api.OP_T, -0.5, A, vx, 2.0, vy, api.R_32F)
    assert st == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    with torch.cuda.stream(side):
        assert api.spmv(handle, api.OP_T, -0.5, A, vx, 2.0, vy, api.R_32F, buf, alg=alg) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert api.spmv(handle, api.OP_T, -0.5, A, vx, 2.0, vy, api.R_32F, buf, alg=alg) == 0
    torch.cuda.synchronize()
    for replay in range(3):
        hx = rng.uniform(-1, 1, a.m).astype(np.float32)
        hy = rng.uniform(-1, 1, a.n).astype(np.float32)
        x.copy_(torch.from_numpy(hx))
        y.copy_(torch.from_numpy(hy))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref, bound = oracle.spmv(True, a.m, a.n, a.base, a.ptr, a.col, a.val, -0.5, 2.0, hx, hy)
        assert_within(y.cpu().numpy(), ref, bound, np.float32, what="replay %d, alg %d" % (replay, alg))
    del graph
    torch.cuda.synchronize()
    handle.destroy()


@pytest.mark.parametrize("analysed", [True, False])
def test_spmm_with_long_rows_replays_in_a_hip_graph(torch_gpu, oracle, analysed):
    """Rows of thousands of nonzeros: the list of their pieces is rebuilt by every call (a kernel clears its counters,
    not a memset), the pieces and the sums of the partial sums are kernels.  analysed: an eager call has left the
    row lengths on the descriptor; else the captured call is the first on the structure, cannot read them back and
    takes the launches for long rows without knowing whether there are any."""
    torch = torch_gpu
    rng = np.random.default_rng(24)
    side = torch.cuda.Stream()
    handle = api.Handle(stream=side.cuda_stream)
    a = wl.mixed_rows(m=6000, per_row=9, long_rows=5, long_len=9000, dtype=np.float64)
    n = 24
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    A = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    B = torch.zeros((a.n, n), dtype=torch.float64, device="cuda")
    C = torch.zeros((a.m, n), dtype=torch.float64, device="cuda")
    mB, mC = api.DnMat(a.n, n, n, B), api.DnMat(a.m, n, n, C)
    st, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, 1.5, A, mB, -0.25, mC, api.R_64F)
    assert st == 0
    buf = torch.empty(size, dtype=torch.uint8, device="cuda")
    if analysed:
        with torch.cuda.stream(side):
            assert api.spmm(handle, api.OP_N, api.OP_N, 1.5, A, mB, -0.25, mC, api.R_64F, buf) == 0
        torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert api.spmm(handle, api.OP_N, api.OP_N, 1.5, A, mB, -0.25, mC, api.R_64F, buf) == 0
    torch.cuda.synchronize()
    for replay in range(3):
        hB = rng.uniform(-1, 1, (a.n, n))
        hC = rng.uniform(-1, 1, (a.m, n))
        B.copy_(torch.from_numpy(hB))
        C.copy_(torch.from_numpy(hC))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref, bound = oracle.spmm(a.m, n, a.base, a.ptr, a.col, a.val, 1.5, -0.25, hB.ravel(), n, True, hC.ravel(), n, True)
        assert_within(C.cpu().numpy(), ref, bound, np.float64, what="replay %d, analysed %r" % (replay, analysed))
    del graph
    torch.cuda.synchronize()
    handle.destroy()


def test_static_buffer_call_replays_in_a_hip_graph(torch_gpu, oracle):
    """mcsparseSpMV_staticBuffer is for callers that cannot allocate, code under graph capture among them.  The
    address of its scratch array is looked up at the first call on a device, which a capture cannot hold: that call
    answers NOT_SUPPORTED under capture (and leaves the capture intact), any later one is captured and replays."""
    torch = torch_gpu
    rng = np.random.default_rng(33)
    side = torch.cuda.Stream()
    handle = api.Handle(stream=side.cuda_stream)
    a = wl.power_law(m=5000, max_len=4000, dtype=np.float32)
    d_ptr, d_col, d_val = dev(torch, a.ptr), dev(torch, a.col), dev(torch, a.val)
    mat = api.SpMat(a.m, a.n, a.nnz, d_ptr, d_col, d_val, base=a.base)
    mat.set_plan(api.FAMILY_MERGE)  # the family that uses the scratch; no analysis, which would read back
    x = torch.zeros(a.n, dtype=torch.float32, device="cuda")
    y = torch.zeros(a.m, dtype=torch.float32, device="cuda")
    vx, vy = api.DnVec(x), api.DnVec(y)

    first = torch.cuda.CUDAGraph()
    with torch.cuda.graph(first, stream=side):
        st = api.spmv_static_buffer(handle, api.OP_N, 2.0, mat, vx, 0.0, vy, api.R_32F)
    torch.cuda.synchronize()
    assert st in (api.STATUS_SUCCESS, api.STATUS_NOT_SUPPORTED)  # SUCCESS when an earlier test made the first call
    del first

    with torch.cuda.stream(side):
        assert api.spmv_static_buffer(handle, api.OP_N, 2.0, mat, vx, 0.0, vy, api.R_32F) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert api.spmv_static_buffer(handle, api.OP_N, 2.0, mat, vx, 0.0, vy, api.R_32F) == api.STATUS_SUCCESS
    torch.cuda.synchronize()
    for replay in range(3):
        hx = rng.uniform(-1, 1, a.n).astype(np.float32)
        x.copy_(torch.from_numpy(hx))
        y.fill_(-3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref, bound = oracle.spmv(False, a.m, a.n, a.base, a.ptr, a.col, a.val, 2.0, 0.0, hx, np.zeros(a.m, np.float32))
        assert_within(y.cpu().numpy(), ref, bound, np.float32, what="replay %d, static buffer" % replay)
    del graph
    torch.cuda.synchronize()
    handle.destroy()
