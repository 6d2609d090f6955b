"""The model-level boundary: a plan recorded through the C-ABI and replayed from the reference's packed
`main(void** params)` block (src/Compiler/Execution.cpp:21-66), checked against the C oracle, and the
engine's use of it checked bit for bit against kernel-by-kernel launches."""
import copy
import ctypes

import numpy as np
import pytest
import torch

from tests.util import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_as_close_as_eager, assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")


def _stream():
    from llcompiler_amd import _capi as C
    return C.current_stream(torch.device("cuda", 0))


def _record_two_layer(plan, x, out, w1_host, b1_host, w2_host, hidden):
    """out = relu(x @ w1 + b1) @ w2 with the weights uploaded into the plan and the hidden layer in its arena."""
    from llcompiler_amd import _capi as C
    L = C.lib()
    M, K = x.shape
    N = out.shape[1]

    def fixed(ptr, shape):
        st, s = [], 1
        for d in reversed(shape):
            st.insert(0, s)
            s *= d
        return C.TensorRef(ptr, C.FLOAT32, shape, st)

    w1 = fixed(plan.upload(w1_host.ctypes.data, w1_host.nbytes), (K, hidden))
    b1 = fixed(plan.upload(b1_host.ctypes.data, b1_host.nbytes), (hidden,))
    w2 = fixed(plan.upload(w2_host.ctypes.data, w2_host.nbytes), (hidden, N))
    h = fixed(plan.alloc(M * hidden * 4), (M, hidden))
    plan.declare_io(x, False)
    plan.declare_io(out, True)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    epi = C.LlcEpilogue(1.0, b1.ptr, None, C.ACT_RELU)
    with plan.recording():
        C.check(L.llc_hip_matmul(rx.ptr, w1.ptr, ctypes.pointer(epi), h.ptr, _stream()))
        C.check(L.llc_hip_matmul(h.ptr, w2.ptr, None, ro.ptr, _stream()))


def test_recorded_plan_replays_from_the_packed_block(oracle):
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    rng = np.random.default_rng(7)
    M, K, H, N = 48, 80, 96, 24
    w1 = rng.standard_normal((K, H), dtype=np.float32) * 0.1
    b1 = rng.standard_normal((H,), dtype=np.float32)
    w2 = rng.standard_normal((H, N), dtype=np.float32) * 0.1
    x0 = rng.standard_normal((M, K), dtype=np.float32)

    def want(x):
        return oracle.matmul(oracle.unary("relu", oracle.matmul(x, w1) + b1), w2)

    plan = Plan()
    x = torch.from_numpy(x0).cuda()
    out = torch.empty((M, N), device="cuda")
    _record_two_layer(plan, x, out, w1, b1, w2, H)
    assert plan.num_steps == 2 and plan.num_params == 11
    torch.cuda.synchronize()
    # recording launches too
    assert_close(out.cpu().numpy(), want(x0), F32_RTOL, F32_ATOL, "recording run")
    # replay with other buffers, at other addresses, holding other values
    for seed in (1, 2):
        xs = np.random.default_rng(seed).standard_normal((M, K), dtype=np.float32)
        pad = torch.empty(seed * 1000, device="cuda")  # shifts the next allocations
        x2 = torch.from_numpy(xs).cuda()
        out2 = torch.zeros((M, N), device="cuda")
        assert x2.data_ptr() != x.data_ptr() and out2.data_ptr() != out.data_ptr()
        plan.run(ParamBlock([x2, out2]), _stream())
        torch.cuda.synchronize()
        assert_close(out2.cpu().numpy(), want(xs), F32_RTOL, F32_ATOL, "replay %d" % seed)
        del pad
    # the first buffers were not written again
    assert_close(out.cpu().numpy(), want(x0), F32_RTOL, F32_ATOL, "recording buffers untouched")

    # an input that is a view at an offset inside a larger buffer: data_ptr carries the offset, slot 2 holds 0
    big = torch.zeros((M + 3, K), device="cuda")
    big[3:] = torch.from_numpy(x0).cuda()
    out3 = torch.zeros((M, N), device="cuda")
    plan.run(ParamBlock([big[3:], out3]), _stream())
    torch.cuda.synchronize()
    assert_close(out3.cpu().numpy(), want(x0), F32_RTOL, F32_ATOL, "replay from a view")

    # the offset slot is honoured like the reference's descriptor offset (Tensor.h:42-47), in elements
    blk = ParamBlock([big, out3])
    off = ctypes.c_size_t(3 * K)
    size = (ctypes.c_size_t * 2)(M, K)
    blk.arr[3] = ctypes.addressof(off)
    blk.arr[4] = ctypes.addressof(size)
    out3.zero_()
    plan.run(blk, _stream())
    torch.cuda.synchronize()
    assert_close(out3.cpu().numpy(), want(x0), F32_RTOL, F32_ATOL, "replay with an element offset")


def test_plan_refuses_other_extents_strides_and_symbols():
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    rng = np.random.default_rng(3)
    M, K, H, N = 16, 32, 32, 8
    plan = Plan()
    x = torch.zeros((M, K), device="cuda")
    out = torch.empty((M, N), device="cuda")
    plan.expect_symbols([M])
    _record_two_layer(plan, x, out, rng.standard_normal((K, H), dtype=np.float32), np.zeros(H, np.float32),
                      rng.standard_normal((H, N), dtype=np.float32), H)
    with pytest.raises(C.LlcHipError) as e:  # slot 0 is NULL but the plan expects a symbol
        plan.run(ParamBlock([x, out]), _stream())
    assert e.value.status == C.ERR_BAD_ARG
    with pytest.raises(C.LlcHipError) as e:
        plan.run(ParamBlock([x, out], symbols=[M + 1]), _stream())
    assert e.value.status == C.ERR_SHAPE
    plan.run(ParamBlock([x, out], symbols=[M]), _stream())
    with pytest.raises(C.LlcHipError) as e:
        plan.run(ParamBlock([torch.zeros((M + 1, K), device="cuda"), out], symbols=[M]), _stream())
    assert e.value.status == C.ERR_SHAPE
    with pytest.raises(C.LlcHipError) as e:
        plan.run(ParamBlock([torch.zeros((K, M), device="cuda").t(), out], symbols=[M]), _stream())
    assert e.value.status == C.ERR_LAYOUT
    # a plan is recorded once, and ops outside begin/end are not recorded
    assert C.lib().llc_plan_begin(plan.handle) == C.ERR_BAD_ARG
    assert plan.num_steps == 2
    torch.cuda.synchronize()


def test_entry_library_main_runs_the_bound_plan(oracle):
    """What Execution::run does (Execution.cpp:12-16, 21-66): resolve `main`, call it with the packed block."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    rng = np.random.default_rng(11)
    M, K, H, N = 8, 784, 512, 10  # the reference's own MLP case, batch 8
    w1 = rng.standard_normal((K, H), dtype=np.float32) * 0.02
    b1 = rng.standard_normal((H,), dtype=np.float32) * 0.02
    w2 = rng.standard_normal((H, N), dtype=np.float32) * 0.02
    plan = Plan()
    x = torch.zeros((M, K), device="cuda")
    out = torch.empty((M, N), device="cuda")
    _record_two_layer(plan, x, out, w1, b1, w2, H)
    L = C.lib()
    E = ctypes.CDLL(C.ENTRY_LIB_PATH)
    E.main.restype = None
    E.main.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    C.check(L.llc_hip_bind_entry(plan.handle, _stream()))
    try:
        xs = rng.standard_normal((M, K), dtype=np.float32)
        x2 = torch.from_numpy(xs).cuda()
        out2 = torch.zeros((M, N), device="cuda")
        blk = ParamBlock([x2, out2])
        E.main(blk.arr)
        assert L.llc_hip_entry_status() == 0
        torch.cuda.synchronize()
        want = oracle.matmul(oracle.unary("relu", oracle.matmul(xs, w1) + b1), w2)
        assert_close(out2.cpu().numpy(), want, F32_RTOL, F32_ATOL, "main(void**)")
    finally:
        C.check(L.llc_hip_bind_entry(None, None))
    E.main(blk.arr)  # nothing bound: logged, status kept, no launch
    assert L.llc_hip_entry_status() == C.ERR_BAD_ARG


def _run_both_ways(build, calls):
    """Runs `calls` (a list of argument tuples) through two engines built by `build`, one replaying native plans,
    one launching kernel by kernel; returns the two lists of results."""
    from llcompiler_amd.executor import engine as E
    got = []
    for use_plan in (True, False):
        E.USE_PLAN = use_plan
        try:
            fn = build()
            with torch.no_grad():
                got.append([fn(*a).clone() for a in calls])
        finally:
            E.USE_PLAN = True
    torch.cuda.synchronize()
    return got


def test_engine_plan_replay_matches_kernel_by_kernel_launches_encoder():
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import EncoderBlock, make_encoder_inputs
    enc = EncoderBlock().eval().to(torch.bfloat16)
    ref = copy.deepcopy(enc).float()
    (x8,) = make_encoder_inputs(2, 128, dtype=torch.bfloat16)

    def build():
        return compile_module(copy.deepcopy(enc).cuda(), (x8.cuda(),), dynamic_shapes=({0: torch.export.Dim("batch")},))

    calls = []
    for B, seed in ((2, 0), (2, 1), (3, 2), (2, 3), (3, 4)):  # first calls record, later ones replay
        (x,) = make_encoder_inputs(B, 128, seed=seed, dtype=torch.bfloat16)
        calls.append((x.cuda(),))
    planned, direct = _run_both_ways(build, calls)
    for (x,), a, b in zip(calls, planned, direct):
        assert torch.equal(a, b)
        xc = x.cpu()
        with torch.no_grad():
            assert_as_close_as_eager(a.float().cpu().numpy(), enc(xc).float().numpy(), ref.double()(xc.double()).numpy(),
                                     BF16_RTOL, BF16_ATOL, "encoder via plan")


def test_engine_plan_replay_matches_kernel_by_kernel_launches_resnet():
    from llcompiler_amd import LLCompiler
    from llcompiler_amd.test_models import ResNet18Folded, make_resnet_inputs
    m = ResNet18Folded().eval()

    def build():
        torch._dynamo.reset()
        comp = LLCompiler(mode="inference", target="gfx950", pipeline="hip")
        return torch.compile(copy.deepcopy(m).cuda(), backend=comp, dynamic=False, fullgraph=True)

    calls = [(make_resnet_inputs(2, 64, seed=s)[0].cuda(),) for s in (0, 1, 2)]
    planned, direct = _run_both_ways(build, calls)
    with torch.no_grad():
        for (x,), a, b in zip(calls, planned, direct):
            assert torch.equal(a, b)
            assert_close(a.cpu().numpy(), m(x.cpu()).numpy(), F32_RTOL, F32_ATOL, "resnet via plan")


def test_engine_inputs_that_stop_sharing_memory_get_their_own_instance(oracle):
    """An instance binds descriptors to inputs by address; two inputs that are views of one buffer in the
    recording call and separate tensors later must not be confused."""
    from llcompiler_amd.compiler.aot import compile_module

    class AddMul(torch.nn.Module):
        def forward(self, a, b):
            return torch.relu(a * 2.0 + b)

    both = torch.arange(32, dtype=torch.float32, device="cuda").reshape(2, 16) - 10.0
    cm = compile_module(AddMul().cuda(), (both[0], both[1]))
    r1 = cm(both[0], both[1])
    r1b = cm(both[0], both[1])
    a = torch.full((16,), 3.0, device="cuda")
    b = torch.full((16,), -5.0, device="cuda")
    r2 = cm(a, b)       # same shapes and strides, no shared memory
    r2b = cm(a, b)
    r3 = cm(both[0], both[1])
    r4 = cm(a, a)       # one tensor twice ...
    r5 = cm(a, b)       # ... and apart again
    r6 = cm(b, b)
    torch.cuda.synchronize()
    w = both.cpu().numpy()
    want1 = oracle.unary("relu", w[0] * 2.0 + w[1])
    for r in (r1, r1b, r3):
        np.testing.assert_array_equal(r.cpu().numpy(), want1)
    for r in (r2, r2b, r5):
        np.testing.assert_array_equal(r.cpu().numpy(), np.full(16, 1.0, np.float32))
    np.testing.assert_array_equal(r4.cpu().numpy(), np.full(16, 9.0, np.float32))
    np.testing.assert_array_equal(r6.cpu().numpy(), np.full(16, 0.0, np.float32))


def test_npy_weights_are_uploaded_into_the_plan(oracle, tmp_path):
    """llh.weight: a .npy file (np.save, as the reference's importer writes it) read by the library into plan-owned
    memory, then used by a recorded plan."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    rng = np.random.default_rng(5)
    M, K, N = 24, 40, 56
    w = rng.standard_normal((K, N), dtype=np.float32)
    path = str(tmp_path / "w.npy")
    np.save(path, w)
    plan = Plan()
    ptr, code, shape = plan.load_npy(path, C.FLOAT32)
    assert (code, shape) == (C.FLOAT32, (K, N)) and ptr
    with pytest.raises(C.LlcHipError):
        plan.load_npy(path, C.INT64)
    wref = C.TensorRef(ptr, C.FLOAT32, (K, N), (N, 1))
    x = torch.from_numpy(rng.standard_normal((M, K), dtype=np.float32)).cuda()
    out = torch.empty((M, N), device="cuda")
    plan.declare_io(x, False)
    plan.declare_io(out, True)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    with plan.recording():
        C.check(C.lib().llc_hip_matmul(rx.ptr, wref.ptr, None, ro.ptr, _stream()))
    xs = rng.standard_normal((M, K), dtype=np.float32)
    out2 = torch.zeros((M, N), device="cuda")
    plan.run(ParamBlock([torch.from_numpy(xs).cuda(), out2]), _stream())
    torch.cuda.synchronize()
    assert_close(out2.cpu().numpy(), oracle.matmul(xs, w), F32_RTOL, F32_ATOL, "matmul with a .npy weight")


def test_models_with_npy_weights_match_models_with_tensor_weights(tmp_path):
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import MLP, EncoderBlock, make_encoder_inputs, make_mlp_inputs
    with torch.no_grad():
        m = MLP().eval().cuda()
        (x,) = make_mlp_inputs()
        a = compile_module(m, (x.cuda(),))
        b = compile_module(m, (x.cuda(),), weights="npy", weight_dir=str(tmp_path / "mlp"))
        assert b.lifted == [] and len(b.engine.graph.inputs) == 1
        for seed in (1, 2, 3):
            (xs,) = make_mlp_inputs(seed=seed)
            assert torch.equal(a(xs.cuda()), b(xs.cuda()))
        enc = EncoderBlock(hidden=128, heads=2, ffn=256).eval().to(torch.bfloat16).cuda()   # bf16 travels as '<u2'
        (xe,) = make_encoder_inputs(2, 64, 128, dtype=torch.bfloat16)
        ea = compile_module(enc, (xe.cuda(),))
        eb = compile_module(enc, (xe.cuda(),), weights="npy", weight_dir=str(tmp_path / "enc"))
        for seed in (1, 2):
            (xs,) = make_encoder_inputs(2, 64, 128, seed=seed, dtype=torch.bfloat16)
            assert torch.equal(ea(xs.cuda()), eb(xs.cuda()))


def test_plan_file_round_trip(oracle, tmp_path):
    """A recorded plan written to a file and read back replays like the original, from memory of its own: the
    uploaded weights travel with their contents, the hidden layer (written before it is read) only by size."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    rng = np.random.default_rng(11)
    M, K, H, N = 40, 72, 2048, 24
    w1 = rng.standard_normal((K, H), dtype=np.float32) * 0.1
    b1 = rng.standard_normal((H,), dtype=np.float32)
    w2 = rng.standard_normal((H, N), dtype=np.float32) * 0.1
    x0 = rng.standard_normal((M, K), dtype=np.float32)
    plan = Plan()
    x = torch.from_numpy(x0).cuda()
    out = torch.empty((M, N), device="cuda")
    _record_two_layer(plan, x, out, w1, b1, w2, H)
    path = tmp_path / "two_layer.llcplan"
    plan.save(path)
    size = path.stat().st_size
    weights = w1.nbytes + b1.nbytes + w2.nbytes
    assert weights < size < weights + 4096, "the file holds the weights and no intermediate (%d bytes)" % size
    loaded = Plan.load(path)
    assert loaded.num_steps == 2 and loaded.num_params == 11
    del plan                                     # the original and its memory go away
    import gc
    gc.collect()
    filler = torch.full((4 * (K * H + H * N),), float("nan"), device="cuda")   # whatever reuses that memory is poison
    for seed in (3, 4):
        xs = np.random.default_rng(seed).standard_normal((M, K), dtype=np.float32)
        x2, out2 = torch.from_numpy(xs).cuda(), torch.zeros((M, N), device="cuda")
        loaded.run(ParamBlock([x2, out2]), _stream())
        torch.cuda.synchronize()
        want = oracle.matmul(oracle.unary("relu", oracle.matmul(xs, w1) + b1), w2)
        assert_close(out2.cpu().numpy(), want, F32_RTOL, F32_ATOL, "loaded plan, seed %d" % seed)
    del filler
    # the loaded plan checks its block like any other
    with pytest.raises(C.LlcHipError):
        loaded.run(ParamBlock([torch.zeros((M + 1, K), device="cuda"), torch.zeros((M, N), device="cuda")]), _stream())
    # files that are not plans
    junk = tmp_path / "junk.llcplan"
    junk.write_bytes(b"LLCPLAN1" + bytes(5))
    with pytest.raises(C.LlcHipError):
        Plan.load(junk)
    cut = tmp_path / "cut.llcplan"
    cut.write_bytes(path.read_bytes()[: size // 2])
    with pytest.raises(C.LlcHipError):
        Plan.load(cut)
    # a damaged description (the part after the weights: steps, operands, offsets) is refused or loads, never
    # crashes the loader; an absurd extent, stride or offset in particular is refused.  Nothing loaded here is run.
    good = path.read_bytes()
    tail = size - 1400
    refused = 0
    for pos in range(tail - tail % 8, size - 8, 8):
        for word in ((1 << 62).to_bytes(8, "little"), (2 ** 64 - 5).to_bytes(8, "little")):
            bad = tmp_path / "bad.llcplan"
            bad.write_bytes(good[:pos] + word + good[pos + 8:])
            try:
                Plan.load(bad)
            except C.LlcHipError:
                refused += 1
    assert refused > 100, refused
    # an operand count that does not fit the step code (replay indexes the operands by position) is refused: the two
    # matmul steps carry five operand records each, behind an empty attribute block (no integers, zeroed convolution
    # and pooling attributes, no program), which is what locates the count in the file
    marker = bytes(8 * (1 + 11 + 11 + 1)) + (5).to_bytes(8, "little")
    counts = []
    at = good.find(marker, size - 1400)
    while at >= 0:
        counts.append(at + len(marker) - 8)
        at = good.find(marker, at + 1)
    assert len(counts) == 2, counts
    for pos in counts:
        for n_op in (1, 2, 4, 6, 13):
            bad = tmp_path / "bad_count.llcplan"
            bad.write_bytes(good[:pos] + n_op.to_bytes(8, "little") + good[pos + 8:])
            with pytest.raises(C.LlcHipError):
                Plan.load(bad)


def test_execution_and_tensor_have_the_reference_binding_surface(oracle, tmp_path):
    """`Execution.load / run / run_with_symbols` and `Tensor(data, base, type, offset, size, stride)` as the
    reference binds them (src/Pybind/Entrance.cpp:70-92,113-119), over a plan file: called the way
    llcompiler/executor/engine.py:34-78 calls them."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.execution import Execution, Tensor
    from llcompiler_amd.executor.plan_runner import Plan
    C.init(0)
    rng = np.random.default_rng(21)
    M, K, H, N = 24, 40, 64, 8
    w1 = rng.standard_normal((K, H), dtype=np.float32) * 0.1
    b1 = rng.standard_normal((H,), dtype=np.float32)
    w2 = rng.standard_normal((H, N), dtype=np.float32) * 0.1
    x = torch.from_numpy(rng.standard_normal((M, K), dtype=np.float32)).cuda()
    out = torch.empty((M, N), device="cuda")
    plan = Plan()
    plan.expect_symbols([M])
    _record_two_layer(plan, x, out, w1, b1, w2, H)
    path = tmp_path / "sym.llcplan"
    plan.save(path)
    del plan

    def trans_to_tensor(*args):  # the reference's own conversion (engine.py:34-54), storage offset 0
        return [Tensor(a.data_ptr(), a.data_ptr() + a.storage_offset(), C.FLOAT32, a.storage_offset(), a.shape, a.stride())
                for a in args]

    ex = Execution()
    with pytest.raises(RuntimeError):
        ex.run(trans_to_tensor(x), trans_to_tensor(out))          # nothing loaded yet
    ex.load(str(path))
    xs = rng.standard_normal((M, K), dtype=np.float32)
    x2, out2 = torch.from_numpy(xs).cuda(), torch.zeros((M, N), device="cuda")
    ex.run_with_symbols([M], trans_to_tensor(x2), trans_to_tensor(out2))
    torch.cuda.synchronize()
    want = oracle.matmul(oracle.unary("relu", oracle.matmul(xs, w1) + b1), w2)
    assert_close(out2.cpu().numpy(), want, F32_RTOL, F32_ATOL, "Execution.run_with_symbols")
    with pytest.raises(C.LlcHipError):
        ex.run_with_symbols([M + 1], trans_to_tensor(x2), trans_to_tensor(out2))   # not the binding it was recorded for
    with pytest.raises(C.LlcHipError):
        ex.run(trans_to_tensor(x2), trans_to_tensor(out2))                         # the plan expects its symbol values
    with pytest.raises(ValueError):
        ex.run_with_symbols([M], trans_to_tensor(x2, x2), trans_to_tensor(out2))
    # a second object with the same file is independent of the first (no process-wide binding)
    ex2 = Execution()
    ex2.load(str(path))
    out3 = torch.zeros((M, N), device="cuda")
    ex2.run_with_symbols([M], trans_to_tensor(x2), trans_to_tensor(out3))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out3.cpu().numpy(), out2.cpu().numpy())


def test_two_plans_with_split_reductions_run_on_two_streams_at_once():
    """Each plan owns the scratch memory of its split reductions: two plans replayed at the same time on two streams
    give, bit for bit, what each gives alone (with one scratch buffer per device they overwrote each other's partial
    sums)."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    L = C.lib()
    M, N, K = 1024, 768, 3072                       # few output tiles, long reduction: split into chunks
    gen = torch.Generator().manual_seed(5)
    plans, blocks, outs = [], [], []
    for _ in range(2):
        a = (torch.rand(M, K, generator=gen) * 2 - 1).cuda()
        w = (torch.rand(N, K, generator=gen) * 2 - 1).cuda()
        out = torch.empty((M, N), device="cuda")
        plan = Plan()
        plan.declare_io(a, False)
        plan.declare_io(w, False)
        plan.declare_io(out, True)
        ra, rw, ro = C.tensor_ref(a), C.tensor_ref(w.t()), C.tensor_ref(out)
        with plan.recording():
            C.check(L.llc_hip_matmul(ra.ptr, rw.ptr, None, ro.ptr, _stream()))
        plans.append(plan)
        blocks.append(ParamBlock([a, w, out]))
        outs.append(out)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    alone = []
    for plan, block, out, st in zip(plans, blocks, outs, streams):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        plan.run(block, st.cuda_stream)
        torch.cuda.synchronize()
        alone.append(out.clone())
        assert not torch.isnan(out).any()
    for out in outs:
        out.fill_(float("nan"))
    torch.cuda.synchronize()
    for _ in range(10):
        for plan, block, st in zip(plans, blocks, streams):
            plan.run(block, st.cuda_stream)
    torch.cuda.synchronize()
    for out, want in zip(outs, alone):
        np.testing.assert_array_equal(out.cpu().numpy(), want.cpu().numpy())


def test_a_plan_refuses_tensors_at_another_alignment_and_the_engine_relaunches_kernel_by_kernel():
    """Kernels and scratch memory of a plan are chosen for the 16-byte alignment class of the tensors it was recorded
    with (a misaligned operand takes no split reduction and needs no scratch memory; an aligned one does): llc_hip_run
    refuses a tensor at another address modulo 16 with LLC_ERR_LAYOUT, and the engine then launches that call's kernels
    one by one, which choose again."""
    from llcompiler_amd import _capi as C
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    C.init(0)
    L = C.lib()
    M, N, K = 512, 768, 3072
    gen = torch.Generator().manual_seed(7)
    w = (torch.rand(N, K, generator=gen) * 2 - 1).cuda()
    base = (torch.rand(M * K + 8, generator=gen) * 2 - 1).cuda()
    odd = base[1:1 + M * K].view(M, K)         # 4 bytes past a 16-byte boundary
    even = base[4:4 + M * K].view(M, K)
    assert odd.data_ptr() % 16 == 4 and even.data_ptr() % 16 == 0
    out = torch.empty((M, N), device="cuda")
    plan = Plan()
    for t, is_out in ((odd, False), (w, False), (out, True)):
        plan.declare_io(t, is_out)
    with plan.recording():
        C.check(L.llc_hip_matmul(C.tensor_ref(odd).ptr, C.tensor_ref(w.t()).ptr, None, C.tensor_ref(out).ptr, _stream()))
    torch.cuda.synchronize()
    want_odd = out.clone()
    with pytest.raises(C.LlcHipError) as err:
        plan.run(ParamBlock([even, w, out]), _stream())
    assert err.value.status == C.ERR_LAYOUT and "modulo 16" in str(err.value)
    out.fill_(float("nan"))
    plan.run(ParamBlock([odd, w, out]), _stream())
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), want_odd.cpu().numpy())

    class Lin(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = torch.nn.Linear(K, N, bias=False)

        def forward(self, x):
            return self.fc(x)

    m = Lin().eval().cuda()
    with torch.no_grad():
        cm = compile_module(m, (even,))
        first = cm(even)
        assert torch.equal(cm(even), first)                      # the recorded plan
        got_odd = cm(odd)                                        # same shape and strides, another alignment class
        assert len(cm.engine.instances) == 1
        torch.testing.assert_close(got_odd, m(odd), rtol=1e-4, atol=1e-4)
        assert torch.equal(cm(even), first)


def test_op_calls_with_split_reductions_run_on_two_streams_at_once():
    """Op entry points called outside a plan keep the partial sums of a split reduction in a scratch buffer per
    (device, stream): the same product issued on two streams at the same time gives, bit for bit, what each call
    gives alone.  llc_hip_scratch_bytes sees one live buffer per stream; llc_hip_trim hands the memory back."""
    import ctypes
    from llcompiler_amd import _capi as C
    C.init(0)
    L = C.lib()
    M, N, K = 1024, 768, 3072
    gen = torch.Generator().manual_seed(6)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    sets = []
    for _ in range(2):
        a = (torch.rand(M, K, generator=gen) * 2 - 1).cuda()
        w = (torch.rand(N, K, generator=gen) * 2 - 1).cuda()
        out = torch.empty((M, N), device="cuda")
        sets.append((C.tensor_ref(a), C.tensor_ref(w.t()), C.tensor_ref(out), out))
    torch.cuda.synchronize()
    alone = []
    for (ra, rw, ro, out), st in zip(sets, streams):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        C.check(L.llc_hip_matmul(ra.ptr, rw.ptr, None, ro.ptr, ctypes.c_void_p(st.cuda_stream)))
        torch.cuda.synchronize()
        assert not torch.isnan(out).any()
        alone.append(out.clone())
    live, retired = ctypes.c_size_t(0), ctypes.c_size_t(0)
    C.check(L.llc_hip_scratch_bytes(0, ctypes.byref(live), ctypes.byref(retired)))
    assert live.value >= 2 * 2 * M * N * 4      # each stream holds its own buffer of at least two chunks of partial sums
    for *_, out in sets:
        out.fill_(float("nan"))
    torch.cuda.synchronize()
    for _ in range(10):
        for (ra, rw, ro, out), st in zip(sets, streams):
            C.check(L.llc_hip_matmul(ra.ptr, rw.ptr, None, ro.ptr, ctypes.c_void_p(st.cuda_stream)))
    torch.cuda.synchronize()
    for (*_, out), want in zip(sets, alone):
        np.testing.assert_array_equal(out.cpu().numpy(), want.cpu().numpy())
    C.check(L.llc_hip_trim(1))
    C.check(L.llc_hip_scratch_bytes(0, ctypes.byref(live), ctypes.byref(retired)))
    assert live.value == 0 and retired.value == 0
    # and the next call allocates again
    ra, rw, ro, out = sets[0]
    C.check(L.llc_hip_matmul(ra.ptr, rw.ptr, None, ro.ptr, ctypes.c_void_p(streams[0].cuda_stream)))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), alone[0].cpu().numpy())


@pytest.mark.parametrize("which", ["encoder_bf16", "resnet"])
def test_engine_plans_survive_a_file(which, tmp_path):
    """The plan an engine instance records (fused attention, stacked projections, channels-last convolutions with
    their prepared weight copies, constants) written to a file and read back gives the engine's result bit for bit."""
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
    from llcompiler_amd.test_models import EncoderBlock, ResNet18Folded, make_encoder_inputs, make_resnet_inputs
    if which == "resnet":
        m = ResNet18Folded().eval().cuda()
        (x,) = make_resnet_inputs(2, 64)
        x = x.cuda()
    else:
        m = EncoderBlock().eval().to(torch.bfloat16).cuda()
        x = make_encoder_inputs(2, 128)[0].to(torch.bfloat16).cuda()
    with torch.no_grad():
        cm = compile_module(m, (x,))
        cm(x)
        inst = list(cm.engine.instances.values())[0]
        seen, run = {}, inst.run

        def spy(inputs):                               # the tensors of the block: lifted parameters, then x
            seen["inputs"] = list(inputs)
            return run(inputs)
        inst.run = spy
        want = cm(x)                                   # second run: the recorded plan
        assert inst._plan is not None and seen["inputs"][-1] is x
        path = tmp_path / (which + ".llcplan")
        inst._plan.save(path)
        loaded = Plan.load(path)
        assert loaded.num_steps == inst._plan.num_steps
    blk_inputs = seen["inputs"]
    out = torch.zeros_like(want)
    loaded.run(ParamBlock(list(blk_inputs) + [out]), _stream())
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    # intermediates are not in the file: it is smaller than the weights' prepared copies plus a margin
    n_param_bytes = sum(p.numel() * p.element_size() for p in m.parameters())
    assert path.stat().st_size < n_param_bytes + (4 << 20)


_RUN_PLAN_FILE = '''
import json, sys
import numpy as np
import torch
from llcompiler_amd import _capi as C
from llcompiler_amd.executor.plan_runner import ParamBlock, Plan
C.init(0)
path, x_file, out_file = sys.argv[1:4]
meta = json.load(open(path + ".json"))
plan = Plan.load(path)
assert plan.num_steps == meta["steps"]
x = torch.from_numpy(np.load(x_file)).cuda()
assert [list(x.shape)] == [i["shape"] for i in meta["inputs"]]
outs = [torch.empty(o["shape"], dtype=getattr(torch, o["dtype"]), device="cuda") for o in meta["outputs"]]
plan.run(ParamBlock([x] + outs), C.current_stream(torch.device("cuda", 0)))
torch.cuda.synchronize()
np.save(out_file, outs[0].cpu().numpy())
'''


def test_saved_plan_with_baked_weights_runs_in_another_process(tmp_path):
    """Compile with the weights taken from .npy files, save the plan: the file is self-contained (the weights are
    part of it, as in the reference's compiled object) and a fresh process that never saw the model gets the same
    bits from it, given only the input."""
    import os
    import subprocess
    import sys
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import MLP, make_mlp_inputs
    m = MLP().eval().cuda()
    (x,) = make_mlp_inputs(seed=5)
    with torch.no_grad():
        cm = compile_module(m, (x.cuda(),), weights="npy", weight_dir=str(tmp_path / "w"))
        want = cm(x.cuda()).cpu().numpy()
        path = str(tmp_path / "mlp.llcplan")
        meta = cm.save_plan(path, x.cuda())
    assert len(meta["inputs"]) == 1 and len(meta["outputs"]) == 1 and meta["steps"] == 2
    n_weight_bytes = sum(p.numel() * 4 for p in m.parameters())
    assert n_weight_bytes <= os.path.getsize(path) < n_weight_bytes + 8192
    np.save(tmp_path / "x.npy", x.numpy())
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _RUN_PLAN_FILE, path, str(tmp_path / "x.npy"), str(tmp_path / "out.npy")],
                       cwd=root, timeout=110, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    np.testing.assert_array_equal(np.load(tmp_path / "out.npy"), want)
    # and the same file through the host written in plain C (no Python, no torch: the C-ABI alone)
    from llcompiler_amd.build import RUN_PLAN
    assert os.path.exists(RUN_PLAN), "llc_run_plan is built with the library (python -m llcompiler_amd.build)"
    r = subprocess.run([RUN_PLAN, path, str(tmp_path / "x.npy"), "-o", str(tmp_path / "out_c.npy")], timeout=110,
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    np.testing.assert_array_equal(np.load(tmp_path / "out_c.npy"), want)
    r = subprocess.run([RUN_PLAN, path, str(tmp_path / "x.npy"), str(tmp_path / "x.npy"), "-o", str(tmp_path / "o.npy")],
                       timeout=110, capture_output=True, text=True)
    assert r.returncode == 1 and "takes 1 inputs" in r.stderr
