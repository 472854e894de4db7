"""sjvp_bwd_noalloc (the backward with its workspace in a static device array of the library, for
callers that cannot allocate) against sjvp_bwd on the same inputs, through the C ABI: bit-exact, on
two calls in a row of which the second is smaller, so that what the first call left in the shared
array must not matter.  Collected last on purpose."""
import ctypes

import pytest
import torch

from oracle import attn_jvp_oracle as orc

pytestmark = pytest.mark.gpu
GRADS = ("dq", "dk", "dv", "dtq", "dtk", "dtv")


def _call(lib, entry, d, o, to, lse, mu, shape, with_workspace):
    from semicat_amd import _lib
    from semicat_amd.kernels import _ptr, _strides
    B, H, Lq, Lk, D = shape
    grads = tuple(torch.full_like(d[n], float("nan")) for n in ("q", "k", "v", "tq", "tk", "tv"))
    tensors = (d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"], o, to, d["dO"], d["dTO"], *grads)
    args = [*(_ptr(t) for t in tensors[:10]), _ptr(lse), _ptr(mu), *(_ptr(t) for t in tensors[10:])]
    keep = None
    if with_workspace:
        nbytes = lib.sjvp_bwd_workspace_bytes(B, H, Lq, Lk, D, _lib.SJVP_BF16)
        keep = torch.empty((nbytes,), device="cuda", dtype=torch.uint8)
        args += [_ptr(keep), nbytes]
    stream = torch.cuda.current_stream().cuda_stream
    rc = entry(*args, B, H, Lq, Lk, D, _strides(tensors), 0.0, _lib.SJVP_BF16, ctypes.c_void_p(stream))
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    return grads


@pytest.mark.parametrize("shapes", [
    [(2, 3, 300, 260, 64), (1, 2, 130, 200, 64)],    # row + column pair, then a smaller problem
    [(1, 2, 200, 150, 128), (2, 2, 128, 128, 64)],   # D = 128 (paired-wave column launch), then the single launch
])
def test_noalloc_backward_equals_the_workspace_entry_point(shapes):
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from semicat_amd import _lib, kernels
    lib = _lib.load()
    for i, shape in enumerate(shapes):
        B, H, Lq, Lk, D = shape
        print(f"[noalloc] call {i}: B{B} H{H} Lq{Lq} Lk{Lk} D{D}", flush=True)
        x = orc.make_inputs(B, H, Lq, Lk, D, seed=40 + i, tangent_scale=0.3, dtype=torch.bfloat16)
        d = {n: t.cuda() for n, t in x.items()}
        o, to, lse, mu, _ = kernels.attention_jvp_forward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"])
        want = _call(lib, lib.sjvp_bwd, d, o, to, lse, mu, shape, True)
        got = _call(lib, lib.sjvp_bwd_noalloc, d, o, to, lse, mu, shape, False)
        for n, a, b in zip(GRADS, got, want):
            assert torch.isfinite(a.float()).all(), n
            assert torch.equal(a, b), f"call {i}: {n} differs between sjvp_bwd_noalloc and sjvp_bwd"
        ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
        for n, a in zip(GRADS, got):
            assert orc.rel_frobenius(a.cpu(), ref[n]) <= 1e-2, n
        # the host wrapper's spelling of the same call
        via = kernels.attention_jvp_backward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"], o, to, lse, mu,
                                             dO=d["dO"], dTO=d["dTO"], static_scratch=True)
        torch.cuda.synchronize()
        for a, b in zip(via, want):
            assert torch.equal(a, b)


def test_noalloc_backward_replays_in_a_captured_graph():
    """The use the entry point is for: captured in a HIP graph (its first call on the device made
    outside the capture, which is when the array's address is looked up), replayed three times with
    fresh inputs copied in and eager work between the replays; every replay equals the eager sjvp_bwd
    result bit for bit."""
    from semicat_amd import kernels
    B, H, Lq, Lk, D = 2, 3, 260, 200, 64  # the row + column pair: the launches that use the scratch
    names = orc.TENSOR_ORDER
    sets = [orc.make_inputs(B, H, Lq, Lk, D, seed=60 + i, tangent_scale=0.3, dtype=torch.bfloat16) for i in range(3)]
    d = {n: torch.empty_like(sets[0][n], device="cuda") for n in names}
    o, to = torch.empty_like(d["q"]), torch.empty_like(d["q"])
    lse = torch.empty((B, H, kernels.stat_rows(Lq)), device="cuda", dtype=torch.float32)
    mu = torch.empty_like(lse)
    grads = tuple(torch.empty_like(d[n]) for n in ("q", "k", "v", "tq", "tk", "tv"))

    def load(i):
        for n in names:
            d[n].copy_(sets[i][n])

    def step(static):
        kernels.attention_jvp_forward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"], o=o, to=to, lse=lse, mu=mu,
                                      with_li=False)
        kernels.attention_jvp_backward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"], o, to, lse, mu,
                                       dO=d["dO"], dTO=d["dTO"], grads=grads, static_scratch=static)

    eager = []
    for i in range(3):
        load(i)
        step(False)  # sjvp_bwd with a workspace of its own
        torch.cuda.synchronize()
        eager.append([t.clone() for t in grads])
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        load(0)
        step(True)  # first call on the device, outside the capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step(True)
        for i in (1, 2, 0):
            load(i)
            for t in grads:
                t.zero_()
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            for n, got, want in zip(GRADS, grads, eager[i]):
                assert torch.equal(got, want), f"replay on input set {i}: {n} differs from the eager sjvp_bwd"


def test_noalloc_backward_rejects_problems_beyond_its_scratch():
    from semicat_amd import _lib
    lib = _lib.load()
    one = ctypes.c_void_p(16)  # placeholder, never dereferenced: the size check comes before any launch
    strides = (ctypes.c_int64 * 48)(*([0] * 48))
    B, H, Lq = 64, 16, 1025  # 64 * 16 * 1152 rows > 1 Mi
    rc = lib.sjvp_bwd_noalloc(*([one] * 18), B, H, Lq, 128, 64, strides, 0.0, _lib.SJVP_BF16, None)
    assert rc == _lib.SJVP_ERR_SCRATCH
    assert "SJVP_NOALLOC_MAX_ROWS" in _lib.strerror(rc)
