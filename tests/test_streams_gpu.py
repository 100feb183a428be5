"""The backward's side lane (dk/dv beside dq on a second stream) and stream capture.

No counterpart in the reference (its Triton launches are serial on one stream, ops/triton.py:436-459). Checked
here: the two-stream backward and the single-stream one (DSDPA_FLAG_SINGLE_STREAM) give the same gradients; work
on a caller's non-default stream is ordered with what that stream does before and after; a captured HIP graph of
forward + backward replays to the eager result. Bars as in the parity tests: rel = max|x - ref| / max|ref|.
"""
import sys

import numpy as np
import pytest
import torch

from ops import _native
from ops.triton import deform_sdpa_triton

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def rel(a, b):
    a, b = a.detach().double().cpu().numpy(), b.detach().double().cpu().numpy()
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def make(seed, B, V, H, Himg, Wimg, D, P, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    L = Himg * Wimg
    q, k, v, do = (torch.randn(B, V, H, L, D, generator=g).to(dtype).cuda() for _ in range(4))
    c = (torch.rand(B, V, L, V, P, 2, generator=g) * 1.2 - 0.1).cuda()
    return q, k, v, c, do


def c_abi_backward(q, k, v, c, do, Himg, Wimg, flags, stream=None):
    lib = _native.load()
    B, V, H, L, D = q.shape
    P = c.shape[-2]
    code = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[q.dtype]
    sfx = {0: "f32", 1: "bf16", 2: "f16"}[code]
    sp = stream.cuda_stream if stream is not None else None
    out, lse = torch.empty_like(q), torch.empty(B, V, H, L, device="cuda")
    fws = torch.empty(max(lib.dsdpa_fwd_workspace_bytes(code, B, V, H, Himg, Wimg, D, P), 1), dtype=torch.uint8,
                      device="cuda")
    ws = torch.empty(lib.dsdpa_bwd_workspace_bytes(code, B, V, H, Himg, Wimg, D, P, flags), dtype=torch.uint8,
                     device="cuda")
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
    _native.check(getattr(lib, "dsdpa_fwd_" + sfx)(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out.data_ptr(), lse.data_ptr(), fws.data_ptr(),
        B, V, H, Himg, Wimg, D, P, 0.3, None, sp))
    _native.check(getattr(lib, "dsdpa_bwd_" + sfx)(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), c.data_ptr(), out.data_ptr(), lse.data_ptr(), do.data_ptr(),
        dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), None, ws.data_ptr(), B, V, H, Himg, Wimg, D, P, 0.3, None, flags, sp))
    return out, dq, dk, dv, (fws, ws, lse)


# The backward forks only from 2^21 query*samples (B*V*H*L * V*P) up and only on shapes whose planes fit in LDS:
# s51, s53, s54 fork; s52 (gather dq) and s55 (small) run on the caller's stream whatever the flag.
SHAPES = [
    # seed B V H Himg Wimg D   P  dtype
    (51, 2, 6, 3, 18, 18, 32, 32, torch.float32),      # planes in LDS
    (52, 1, 2, 2, 30, 30, 64, 5, torch.float32),       # gather dq
    (53, 2, 4, 8, 16, 16, 64, 32, torch.bfloat16),     # fp32 accumulators in the workspace + casts
    (54, 2, 4, 32, 8, 8, 128, 33, torch.float16),
    (55, 2, 3, 2, 6, 7, 32, 11, torch.float32),        # small
]


@pytest.mark.parametrize("shape", SHAPES, ids=[f"s{s[0]}" for s in SHAPES])
def test_side_lane_matches_single_stream(shape):
    seed, B, V, H, Himg, Wimg, D, P, dtype = shape
    say(f"[case] side lane vs single stream seed={seed} B{B} V{V} H{H} {Himg}x{Wimg} D{D} P{P} {dtype}")
    q, k, v, c, do = make(seed, B, V, H, Himg, Wimg, D, P, dtype)
    one = c_abi_backward(q, k, v, c, do, Himg, Wimg, _native.FLAG_SINGLE_STREAM)
    torch.cuda.synchronize()
    for rep in range(3):                               # repeated: the side lane's events and stream are reused
        two = c_abi_backward(q, k, v, c, do, Himg, Wimg, 0)
        torch.cuda.synchronize()
        tol = 1e-5 if dtype == torch.float32 else 1e-2     # float atomics / one rounding to 16 bits
        assert torch.equal(one[0], two[0]) and torch.equal(one[1], two[1])      # out, dq: no atomics
        assert rel(two[2], one[2]) < tol and rel(two[3], one[3]) < tol


def test_caller_stream_is_ordered_before_and_after():
    """Inputs are produced on the caller's stream right before the call and the gradients consumed on it right
    after, with no synchronisation in between: the side lane's fork and join carry the ordering."""
    say("[case] side lane on a non-default stream")
    q, k, v, c, do = make(61, 2, 6, 4, 18, 18, 32, 32)
    ref = c_abi_backward(q, k, v, c, do, 18, 18, _native.FLAG_SINGLE_STREAM)
    torch.cuda.synchronize()
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        for rep in range(4):
            q2, k2, v2, do2 = (t * 2.0 for t in (q, k, v, do))           # produced on st
            q2, k2, v2, do2 = (t * 0.5 for t in (q2, k2, v2, do2))       # exact: back to the originals
            out, dq, dk, dv, keep = c_abi_backward(q2, k2, v2, c, do2, 18, 18, 0, stream=st)
            sums = [t.double().sum() for t in (dq, dk, dv)]              # consumed on st
    st.synchronize()
    assert torch.equal(dq, ref[1])
    assert rel(dk, ref[2]) < 1e-5 and rel(dv, ref[3]) < 1e-5
    for s_, r_ in zip(sums, (ref[1], ref[2], ref[3])):
        assert abs(s_.item() - r_.double().sum().item()) <= 1e-4 * r_.double().abs().sum().item()


# "slabs": fp32 takes the slab kernels (planes loaded straight into LDS), 16-bit the gather kernels; "windows": planes too
# large for LDS with 64 samples per view: fp32 the window mode of the gather kernels, 16-bit the forward on tiles of 16
# queries with the per-query kernel behind it
@pytest.mark.parametrize("dims", [(2, 3, 4, 10, 9, 32, 13), (2, 4, 16, 12, 12, 32, 32), (1, 2, 2, 22, 24, 64, 16),
                                  (1, 2, 2, 24, 40, 64, 64)], ids=["small", "forking", "slabs", "windows"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_captured_graph_replays_to_the_eager_result(dtype, dims):
    """Forward + backward captured once in a HIP graph (torch.cuda.graph), replayed with new inputs copied into
    the static buffers, with eager work and synchronisations between the replays; every replay is compared
    with an eager call on the same inputs."""
    say(f"[case] graph capture {dtype} {dims}")
    B, V, H, Himg, Wimg, D, P = dims                   # the second: large enough for the backward to fork
    q, k, v, c, do = make(71, B, V, H, Himg, Wimg, D, P, dtype)
    sq, sk, sv = (t.clone().requires_grad_(True) for t in (q, k, v))
    sc, sdo = c.clone(), do.clone()

    def step(a, b_, c_, d_, e_):
        out = deform_sdpa_triton(a, b_, c_, d_, Wimg, Himg, 0.3)
        return (out,) + torch.autograd.grad(out, (a, b_, c_), e_)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside the capture, as torch asks
        for _ in range(2):
            step(sq, sk, sv, sc, sdo)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out, s_dq, s_dk, s_dv = step(sq, sk, sv, sc, sdo)
    torch.cuda.synchronize()
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for rep in range(4):
        q2, k2, v2, c2, do2 = make(80 + rep, B, V, H, Himg, Wimg, D, P, dtype)
        with torch.no_grad():
            for dst, src in ((sq, q2), (sk, k2), (sv, v2), (sc, c2), (sdo, do2)):
                dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        e_out, e_dq, e_dk, e_dv = step(q2.requires_grad_(True), k2.requires_grad_(True), v2.requires_grad_(True),
                                       c2, do2)
        torch.cuda.synchronize()
        assert torch.equal(s_out, e_out) and torch.equal(s_dq, e_dq), f"replay {rep}"
        assert rel(s_dk, e_dk) < tol and rel(s_dv, e_dv) < tol, f"replay {rep}"


def test_two_host_threads_with_their_own_streams():
    """Two host threads run forward + backward at the same time, each on a stream of its own (the library keeps
    one second stream per thread and device); both get the single-stream result."""
    import threading
    say("[case] two host threads")
    cases = [make(91, 2, 4, 16, 12, 12, 32, 32), make(92, 2, 4, 16, 10, 13, 64, 32)]     # (both backwards fork)
    dims = [(12, 12), (10, 13)]
    refs = [c_abi_backward(*cases[i], *dims[i], _native.FLAG_SINGLE_STREAM) for i in range(2)]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def work(i):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for _ in range(8):
                    r = c_abi_backward(*cases[i], *dims[i], 0, stream=st)
            st.synchronize()
            results[i] = r
        except Exception as e:                   # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(2):
        assert results[i] is not None
        assert torch.equal(results[i][0], refs[i][0]) and torch.equal(results[i][1], refs[i][1])
        assert rel(results[i][2], refs[i][2]) < 1e-5 and rel(results[i][3], refs[i][3]) < 1e-5
