"""The sampler's entry point that allocates nothing, called through ctypes and compared with the entry point that
takes a workspace: two calls in a row on one device, the second with fewer rows and a smaller vocabulary, so that
the array inside the library still holds the first call's weights when the second runs."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_FLOATS = 1 << 21      # ATOMA_SAMPLE_STATIC_MAX_FLOATS of csrc/kernels/sample_static.h
TOO_LARGE = -4


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _inputs(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn((rows, vocab), generator=g) * 3.0).cuda()
    # greedy, plain temperature, top-k, top-p, both cuts: one row of each kind, then again
    kinds = [(0.0, 0, 1.0), (0.8, 0, 1.0), (1.3, 40, 1.0), (0.7, 0, 0.9), (1.1, 25, 0.8)]
    temperature = torch.tensor([kinds[r % 5][0] for r in range(rows)], dtype=torch.float32).cuda()
    top_k = torch.tensor([kinds[r % 5][1] for r in range(rows)], dtype=torch.int32).cuda()
    top_p = torch.tensor([kinds[r % 5][2] for r in range(rows)], dtype=torch.float32).cuda()
    uniform = torch.rand((rows,), generator=g).cuda()
    return logits, temperature, top_k, top_p, uniform


def _both(lib, rows, vocab, seed):
    logits, temperature, top_k, top_p, uniform = _inputs(rows, vocab, seed)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for static in (False, True):
        tok = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        lg = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
        if static:
            rc = lib.atoma_sample_static(_ptr(logits), vocab, rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                         _ptr(uniform), _ptr(tok), _ptr(lg), stream)
        else:
            work = torch.empty((rows, vocab), dtype=torch.float32, device="cuda")
            rc = lib.atoma_sample(_ptr(logits), vocab, rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                  _ptr(uniform), _ptr(work), _ptr(tok), _ptr(lg), stream)
        assert rc == 0, f"rc {rc} (static={static}, rows={rows}, vocab={vocab})"
        torch.cuda.synchronize()
        outs.append((tok.cpu(), lg.cpu()))
    return outs, logits.cpu()


def test_sampling_without_allocation_matches_the_workspace_entry_point():
    from atoma_infer_amd.kernels.library import load_hip_module
    lib = load_hip_module("core")
    for f in (lib.atoma_sample, lib.atoma_sample_static, lib.atoma_sample_static_init):
        f.restype = ctypes.c_int
    assert lib.atoma_sample_static_init() == 0
    for rows, vocab, seed in ((10, 50021, 1), (3, 1000, 2)):        # the second call is the smaller one
        print(f"sample_static rows={rows} vocab={vocab}", flush=True)
        ((tok_w, lg_w), (tok_s, lg_s)), logits = _both(lib, rows, vocab, seed)
        assert torch.equal(tok_w, tok_s), (tok_w, tok_s)
        assert torch.equal(lg_w, lg_s)
        assert int(tok_s.min()) >= 0 and int(tok_s.max()) < vocab
        # rows 0 and 5 are greedy: the argmax, so the comparison above is not one of two equal mistakes
        for r in range(0, rows, 5):
            assert int(tok_s[r]) == int(logits[r].argmax())
        assert torch.equal(lg_s, logits[torch.arange(rows), tok_s.long()])


def test_sampling_without_allocation_refuses_what_does_not_fit():
    from atoma_infer_amd.kernels.library import load_hip_module
    lib = load_hip_module("core")
    lib.atoma_sample_static.restype = ctypes.c_int
    rows, vocab = 17, 128256                      # 17 * 128256 > 2^21
    assert rows * vocab > MAX_FLOATS
    dummy = torch.zeros((4,), dtype=torch.float32, device="cuda")     # never read: the call returns before any launch
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.atoma_sample_static(_ptr(dummy), vocab, rows, vocab, _ptr(dummy), _ptr(dummy), _ptr(dummy), _ptr(dummy),
                                 _ptr(dummy), _ptr(dummy), stream)
    assert rc == TOO_LARGE
    torch.cuda.synchronize()


def test_sampling_without_allocation_allocates_nothing_and_can_be_captured():
    """What the entry point is for.  Around a call, after the set-up call, the device's free memory (hipMemGetInfo)
    and torch's own books stay as they were; and the call is recorded into a graph, where an allocating call is an
    error, and replayed with eager work and synchronisation between the replays, every replay checked against the
    workspace entry point."""
    from atoma_infer_amd.kernels.library import load_hip_module
    lib = load_hip_module("core")
    for f in (lib.atoma_sample, lib.atoma_sample_static, lib.atoma_sample_static_init):
        f.restype = ctypes.c_int
    assert lib.atoma_sample_static_init() == 0
    rows, vocab = 6, 7001
    logits, temperature, top_k, top_p, uniform = _inputs(rows, vocab, 9)
    tok = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    lg = torch.zeros((rows,), dtype=torch.float32, device="cuda")
    work = torch.empty((rows, vocab), dtype=torch.float32, device="cuda")
    tok_w, lg_w = torch.empty_like(tok), torch.empty_like(lg)
    torch.cuda.synchronize()

    def static_call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return lib.atoma_sample_static(_ptr(logits), vocab, rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                       _ptr(uniform), _ptr(tok), _ptr(lg), stream)

    def workspace_call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.atoma_sample(_ptr(logits), vocab, rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                _ptr(uniform), _ptr(work), _ptr(tok_w), _ptr(lg_w), stream) == 0

    before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert static_call() == 0
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert after == before, f"memory moved around the call: {before} -> {after}"
    workspace_call()
    torch.cuda.synchronize()
    assert torch.equal(tok, tok_w) and torch.equal(lg, lg_w)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert static_call() == 0
    g = torch.Generator().manual_seed(10)
    for replay in range(4):
        # new inputs in the same buffers, eager work of the program's own, then the replay
        logits.copy_((torch.randn((rows, vocab), generator=g) * 3.0).cuda())
        uniform.copy_(torch.rand((rows,), generator=g).cuda())
        tok.fill_(-1)
        workspace_call()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(tok, tok_w) and torch.equal(lg, lg_w), f"replay {replay}"
        assert int(tok[0]) == int(logits[0].argmax())          # row 0 is greedy
