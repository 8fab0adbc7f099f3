"""The allocation-free entry point (qproj_mul_mat_multi_noalloc) against qproj_mul_mat_multi.

It serves callers that cannot allocate device memory (HIP graph capture, tight serving loops): same kernels, the
call's scratch in a fixed 64 MiB buffer inside the library.  Bar: bit-identical outputs (integer dots and the same
fp32 order on both routes), on calls in a row where the later one is smaller and so leaves stale bytes of the
earlier one in the shared buffer; device memory in use does not change across the calls; a call whose scratch
would not fit is refused before anything is launched."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.fixture(scope="module")
def ctx():
    from magnitude_amd import Context
    assert torch.cuda.is_available(), "these tests need the MI355X"
    c = Context(0)
    yield c
    c.close()


def upload(ctx, qtype, n, k, seed):
    from magnitude_amd import synth
    blocks = synth.random_weight(qtype, n, k, seed=seed, device=torch.device("cuda:0"))
    return ctx.upload_from_device(qtype, k, n, blocks)


CASES = [  # (type, K, rows of the tensors sharing the call, [M of the first call, M of the smaller second call, ...])
    (Q6_K, 14336, (1024,), [16, 5]),             # small-batch kernel, K in chunks: per-chunk results in scratch
    (Q4_K, 4096, (1536, 1536), [16, 3, 1]),      # gate/up style pair; the last call is the decode regime (no scratch)
    (Q4_K, 14336, (1024,), [200, 48, 17]),       # tiled kernel, K cut into stretches: partial tiles in scratch
    (Q6_K, 14336, (512,), [130, 40]),            # tiled Q6_K kernel with stretches
    (Q8_0, 4096, (768,), [96, 64, 7]),           # tiled Q8_0 product, then the small-batch kernel
    (Q4_K, 4096, (1024, 256, 256), [64, 20]),    # q/k/v style launch of three tensors
    (Q6_K, 14336, (4096,), [8, 4]),              # two K chunks that add themselves to rows the quantizer cleared
    (Q4_K, 4096, (4096,), [192, 32, 17]),        # two K stretches of a tile that add themselves, then 32-row passes
]


@pytest.mark.parametrize("qtype,k,ns,ms", CASES)
def test_noalloc_matches_mul_mat_multi_on_calls_in_a_row(ctx, qtype, k, ns, ms):
    from magnitude_amd import ACT_GGML, qproj
    ws = [upload(ctx, qtype, n, k, seed=31 * i + n) for i, n in enumerate(ns)]
    g = torch.Generator(device="cuda").manual_seed(k + len(ns))
    xs = [torch.randn((m, k), generator=g, device="cuda") for m in ms]
    want = [[y.clone() for y in ctx.mul_mat_multi(ws, x, ACT_GGML)] for x in xs]     # grows the context's workspace
    outs = [[torch.full((m, n), float("nan"), device="cuda") for n in ns] for m in ms]
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for x, ys, m in zip(xs, outs, ms):              # back to back, no synchronisation in between
        print(f"noalloc call type {qtype} K {k} N {ns} M {m}", flush=True)
        assert qproj.workspace_bytes(qtype, k, ns, m, ACT_GGML) <= qproj.NOALLOC_SCRATCH_BYTES
        ctx.mul_mat_multi(ws, x, ACT_GGML, outs=ys, sync=False, noalloc=True)
    ctx.sync()
    assert torch.cuda.mem_get_info()[0] == free_before          # nothing was allocated or freed on the way
    for ys, ref, m in zip(outs, want, ms):
        for y, r in zip(ys, ref):
            assert torch.equal(y.view(torch.int32), r.view(torch.int32)), f"M = {m}"
    for w in ws:
        w.free()


def test_noalloc_per32_and_fp32_modes(ctx):
    from magnitude_amd import ACT_F32, ACT_Q8X32
    w = upload(ctx, Q4_K, 640, 4096, seed=5)
    g = torch.Generator(device="cuda").manual_seed(9)
    for act, ms in ((ACT_Q8X32, [192, 70]), (ACT_F32, [3, 1])):
        for m in ms:
            x = torch.randn((m, 4096), generator=g, device="cuda")
            want = ctx.mul_mat_multi([w], x, act)[0]
            got = ctx.mul_mat_multi([w], x, act, noalloc=True)[0]
            assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (act, m)
    w.free()


def test_noalloc_refuses_what_does_not_fit(ctx):
    """4096 tokens against the 14336-wide down projection need 58.7 MB of activation planes plus stretches of K:
    more than the fixed buffer.  The call answers INVALID_ARG, names the sizes, and launches nothing."""
    from magnitude_amd import ACT_GGML, QprojError, qproj
    w = upload(ctx, Q6_K, 256, 14336, seed=6)
    m = 4096
    assert qproj.workspace_bytes(Q6_K, 14336, (256,), m, ACT_GGML) > qproj.NOALLOC_SCRATCH_BYTES
    x = torch.randn((m, 14336), device="cuda")
    y = torch.full((m, 256), 7.0, device="cuda")
    with pytest.raises(QprojError) as e:
        ctx.mul_mat_multi([w], x, ACT_GGML, outs=[y], noalloc=True)
    assert e.value.status == 1 and "fixed buffer holds" in str(e.value)
    ctx.sync()
    assert bool((y == 7.0).all())                                # untouched
    got = ctx.mul_mat_multi([w], x[:64], ACT_GGML, noalloc=True)[0]   # and the entry point still works afterwards
    want = ctx.mul_mat_multi([w], x[:64], ACT_GGML)[0]
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    w.free()


def test_noalloc_scratch_belongs_to_one_context_at_a_time(ctx):
    """Two contexts launch on two streams; their calls would overwrite each other's scratch in the one fixed buffer
    of the GPU with no error anywhere.  The buffer belongs to the first context that uses it until that context is
    destroyed: a second context is refused, and served once the first is gone."""
    from magnitude_amd import ACT_GGML, Context, QprojError
    w = upload(ctx, Q4_K, 512, 4096, seed=8)
    x = torch.randn((8, 4096), device="cuda")
    want = ctx.mul_mat_multi([w], x, ACT_GGML, noalloc=True)[0]           # this module's context owns the buffer
    other = Context(0)
    try:
        w2 = upload(other, Q4_K, 512, 4096, seed=8)
        with pytest.raises(QprojError) as e:
            other.mul_mat_multi([w2], x, ACT_GGML, noalloc=True)
        assert e.value.status == 4 and "another context" in str(e.value)
        got = other.mul_mat_multi([w2], x, ACT_GGML)[0]                    # its allocating route is untouched
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        w2.free()
    finally:
        other.close()
    again = ctx.mul_mat_multi([w], x, ACT_GGML, noalloc=True)[0]
    assert torch.equal(again.view(torch.int32), want.view(torch.int32))
    w.free()
