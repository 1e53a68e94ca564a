"""The entry point that allocates nothing: ``xkv_recon_stage1_static`` keeps the packed copy of ``k_B`` in a static
device array inside the library instead of a caller workspace.  Called through the C ABI (ctypes) and compared with
``xkv_recon_stage1`` on a torch-allocated workspace: same kernels, so the split partials and log-sum-exps must agree
bit for bit - on two calls in a row, the second with a smaller input (the array keeps the first call's contents)."""
from ctypes import c_float, c_int64

import pytest
import torch

from util import gen

pytestmark = pytest.mark.gpu

from kernel_collections_amd import _lib, ops  # noqa: E402
from kernel_collections_amd._lib import dtype_code, kv_operand, ptr, stream_ptr  # noqa: E402


def _call(static, q, kA, kB, vA, S, theta, dev, poison=None):
    b, hq, d = q.shape
    hkv, r = kB.shape[1], kB.shape[2]
    L = kA.shape[1]
    partial = torch.full((b, hq, S, vA.shape[-1]), float("nan"), device=dev)
    lse = torch.full((b, hq, S), float("nan"), device=dev)
    ns = ops.uniform_splits(b, S, dev)
    inv = ops.rope_inv_freq(d, theta, dev)
    a_op = kv_operand(kA, kA.stride(0), kA.stride(1), 0, r)
    v_op = kv_operand(vA, vA.stride(0), vA.stride(1), 0, vA.shape[-1])
    head = [ptr(q), a_op, ptr(kB), c_int64(kB.stride(0)), c_int64(kB.stride(1)), c_int64(kB.stride(2)), v_op,
            ptr(partial), ptr(lse), ptr(None), 0, ptr(ns), ptr(None), b, hq, hkv, L, S, c_float(d ** -0.5), 1, ptr(inv),
            c_int64(0), ptr(None), c_int64(0)]
    tail = [dtype_code(q.dtype), stream_ptr(q)]
    lib = _lib.lib()
    if static:
        rc = lib.xkv_recon_stage1_static(*head, *tail)
        _lib.check(rc, "stage 1")
        torch.cuda.synchronize()
        # the call above was this shape's warm-up (address look-up, LDS attribute); a second one must leave the device's
        # free memory exactly as it found it: nothing is allocated, by the library or behind its back
        free_before = torch.cuda.mem_get_info()[0]
        rc = lib.xkv_recon_stage1_static(*head, *tail)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "xkv_recon_stage1_static changed the device's free memory"
    else:
        nbytes = lib.xkv_recon_workspace_bytes(b, hkv, r, c_int64(kB.stride(0)))
        assert nbytes > 0
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.xkv_recon_stage1(*head, ptr(ws), c_int64(nbytes), *tail)
    _lib.check(rc, "stage 1")
    torch.cuda.synchronize()
    return partial, lse


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_static_scratch_entry_point_matches_the_workspace_one(dev, dtype):
    theta = 5e5
    # first call: the wave-specialised kernel (rank 512, shared basis), per-sequence factors -> 2 MiB of the 4 MiB array;
    # second call, smaller: the 8-wave kernel (rank 384 keys, rank 256 values), one factor for the batch -> 768 KiB
    shapes = [dict(b=2, hq=32, hkv=8, L=2100, rk=512, rv=512, shared=True, S=3, expand=False),
              dict(b=3, hq=16, hkv=4, L=700, rk=384, rv=256, shared=False, S=2, expand=True)]
    for n, c in enumerate(shapes):
        q = gen((c["b"], c["hq"], 128), std=0.5, dtype=dtype, seed=10 + n).to(dev)
        kA = gen((c["b"], c["L"], c["rk"]), dtype=dtype, seed=20 + n).to(dev)
        vA = kA if c["shared"] else gen((c["b"], c["L"], c["rv"]), dtype=dtype, seed=30 + n).to(dev)
        if c["expand"]:
            kB = gen((1, c["hkv"], c["rk"], 128), std=c["rk"] ** -0.5, dtype=dtype, seed=40 + n).to(dev).expand(c["b"], -1, -1, -1)
        else:
            kB = gen((c["b"], c["hkv"], c["rk"], 128), std=c["rk"] ** -0.5, dtype=dtype, seed=40 + n).to(dev)
        want = _call(False, q, kA, kB, vA, c["S"], theta, dev)
        got = _call(True, q, kA, kB, vA, c["S"], theta, dev)
        assert not torch.isnan(got[1]).any() and torch.equal(got[1], want[1]), f"call {n}: log-sum-exp differs"
        assert torch.equal(got[0], want[0]), f"call {n}: partial outputs differ"


def test_static_scratch_rejects_what_does_not_fit(dev):
    dtype = torch.bfloat16
    b, hq, hkv, L, r = 8, 32, 8, 64, 512          # 8 per-sequence copies of 1 MiB > 4 MiB
    q, kA = gen((b, hq, 128), dtype=dtype).to(dev), gen((b, L, r), dtype=dtype).to(dev)
    kB = gen((b, hkv, r, 128), std=r ** -0.5, dtype=dtype).to(dev)
    assert _lib.lib().xkv_recon_workspace_bytes(b, hkv, r, c_int64(kB.stride(0))) > _lib.STATIC_SCRATCH_BYTES
    with pytest.raises(RuntimeError, match="static device array"):
        _call(True, q, kA, kB, kA, 1, 5e5, dev)


def test_static_scratch_entry_point_under_graph_capture(dev):
    """What the entry point is for: after one warm-up call per shape it can be recorded into a HIP graph (nothing in it
    allocates, looks up symbols or sets attributes any more).  The graph - stage 1 into fixed workspaces, then the merge - is
    replayed three times with new queries in the captured input buffer, with eager work and synchronisations between the
    replays, and every replay is compared with the eager result for the same query."""
    dtype, theta = torch.bfloat16, 5e5
    b, hq, hkv, L, r, S, d = 2, 32, 8, 1500, 512, 3, 128
    kA = gen((b, L, r), dtype=dtype, seed=51).to(dev)
    kB = gen((1, hkv, r, d), std=r ** -0.5, dtype=dtype, seed=52).to(dev).expand(b, -1, -1, -1)
    vB = gen((1, hkv, r, d), std=r ** -0.5, dtype=dtype, seed=53).to(dev).expand(b, -1, -1, -1)
    q_in = torch.zeros((b, hq, d), dtype=dtype, device=dev)
    partial = torch.zeros((b, hq, S, r), device=dev)
    lse = torch.zeros((b, hq, S), device=dev)
    out = torch.zeros((b, hq, d), dtype=dtype, device=dev)
    ns = ops.uniform_splits(b, S, dev)
    inv = ops.rope_inv_freq(d, theta, dev)
    lib = _lib.lib()

    def step():
        a_op = kv_operand(kA, kA.stride(0), kA.stride(1), 0, r)
        rc = lib.xkv_recon_stage1_static(ptr(q_in), a_op, ptr(kB), c_int64(kB.stride(0)), c_int64(kB.stride(1)),
                                         c_int64(kB.stride(2)), a_op, ptr(partial), ptr(lse), ptr(None), 0, ptr(ns), ptr(None),
                                         b, hq, hkv, L, S, c_float(d ** -0.5), 1, ptr(inv), c_int64(0), ptr(None), c_int64(0),
                                         dtype_code(dtype), stream_ptr(q_in))
        _lib.check(rc, "stage 1")
        ops.merge_stage2(partial, lse, out, vB, ns, None, b, hq, hkv, L, S)

    queries = [gen((b, hq, d), std=0.5, dtype=dtype, seed=60 + i).to(dev) for i in range(4)]
    q_in.copy_(queries[0])
    step()                                   # warm-up of this shape, outside the capture
    torch.cuda.synchronize()
    eager = []
    for qq in queries:
        q_in.copy_(qq)
        step()
        eager.append(out.clone())
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        q_in.copy_(queries[0])
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for i in (1, 2, 3):
        q_in.copy_(queries[i])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[i]), f"replay {i} differs from the eager call"
        scratch = torch.randn(1 << 16, device=dev).sum().item()   # eager work between the replays
        assert scratch == scratch
