"""The decode attention entry point that allocates nothing, called through ctypes, against
the entry point that takes its partial sums from the caller: two calls in a row, the second
with a smaller input, so that what the first call left in the library's own buffer is there
when the second runs."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

STATIC_FLOATS = 4 * 1024 * 1024
ERR_SCRATCH = 3


def _lib():
    from return_amd.kernels import build
    lib = ctypes.CDLL(build.ensure_built())
    P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    lib.ra_attention_decode_bf16.argtypes = [P] * 12 + [I] * 5 + [F] + [I] * 4 + [P]
    lib.ra_attention_decode_bf16.restype = I
    lib.ra_attention_decode_static_bf16.argtypes = [P] * 10 + [I] * 5 + [F] + [I] * 4 + [P]
    lib.ra_attention_decode_static_bf16.restype = I
    return lib


def _case(lengths, Hq, Hkv, D, P, split, seed):
    """Requests of the given lengths (the new token's key is already in the cache) on scattered pages."""
    g = torch.Generator().manual_seed(seed)
    need = [-(-n // P) for n in lengths]
    order = torch.randperm(sum(need) + 2, generator=g).tolist()
    table, cu_pages = [], [0]
    for k in need:
        table += [order.pop() for _ in range(k)]
        cu_pages.append(len(table))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    bf = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(DEV)
    n = len(lengths)
    return dict(q=bf(n, Hq, D), kp=bf(sum(need) + 2, Hkv, P, D), vp=bf(sum(need) + 2, Hkv, P, D),
                page_table=i32(table), cu_pages=i32(cu_pages), kv_start=i32([0] * n),
                cu_q=i32(list(range(n + 1))), q_start=i32([m - 1 for m in lengths]), n=n, Hq=Hq, Hkv=Hkv, D=D,
                P=P, split=split, max_splits=(max(lengths) - 1) // split + 1)


def _run(lib, c, static, warm=False):
    out = torch.zeros_like(c["q"])
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    tabs = [p(c["page_table"]), p(c["cu_pages"]), p(c["kv_start"]), p(c["cu_q"]), p(c["q_start"]), None]
    tail = [c["n"], c["Hq"], c["Hkv"], c["D"], c["P"], c["D"] ** -0.5, 0, c["split"], c["max_splits"], 0,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)]
    if static:
        held, free = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = lib.ra_attention_decode_static_bf16(p(c["q"]), p(out), p(c["kp"]), p(c["vp"]), *tabs, *tail)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == held          # nothing through torch's allocator
        if warm:
            assert torch.cuda.mem_get_info()[0] == free       # and nothing beside it, once the kernels are loaded
    else:
        acc = torch.empty(c["n"], c["Hq"], c["max_splits"], c["D"], dtype=torch.float32, device=DEV)
        ml = torch.empty(c["n"], c["Hq"], c["max_splits"], 2, dtype=torch.float32, device=DEV)
        rc = lib.ra_attention_decode_bf16(p(c["q"]), p(out), p(acc), p(ml), p(c["kp"]), p(c["vp"]), *tabs, *tail)
    torch.cuda.synchronize()
    return rc, out


def _plain(c, lengths):
    """Softmax attention of every request's one query over its keys, gathered from the pages, in 32-bit."""
    out = torch.zeros(c["n"], c["Hq"], c["D"])
    kp, vp, table = c["kp"].float().cpu(), c["vp"].float().cpu(), c["page_table"].cpu().tolist()
    q, cu, P, G = c["q"].float().cpu(), c["cu_pages"].cpu().tolist(), c["P"], c["Hq"] // c["Hkv"]
    for i, n in enumerate(lengths):
        pages = table[cu[i]:cu[i + 1]]
        k = torch.cat([kp[p] for p in pages], dim=1)[:, :n]            # [Hkv, n, D]
        v = torch.cat([vp[p] for p in pages], dim=1)[:, :n]
        for h in range(c["Hq"]):
            w = ((k[h // G] @ q[i, h]) * c["D"] ** -0.5).softmax(0)
            out[i, h] = w @ v[h // G]
    return out


def test_decode_attention_without_allocation_two_calls_in_a_row():
    torch.cuda.set_device(0)
    lib = _lib()
    lengths = {"big": [900, 130, 64, 517, 1, 333], "small": [70, 200]}
    big = _case(lengths["big"], Hq=8, Hkv=2, D=128, P=16, split=128, seed=1)
    small = _case(lengths["small"], Hq=6, Hkv=3, D=64, P=16, split=64, seed=2)
    for name, c in (("big", big), ("small", small)):   # the second call finds the first one's partial sums in the buffer
        rc, want = _run(lib, c, static=False)
        assert rc == 0
        rc, got = _run(lib, c, static=True, warm=c is small)
        assert rc == 0
        assert torch.equal(got, want)
        assert want.float().abs().max() > 0
        # and both against a 32-bit evaluation that shares nothing with the library
        torch.testing.assert_close(got.float().cpu(), _plain(c, lengths[name]), atol=2e-2, rtol=2e-2)


def test_decode_attention_without_allocation_refuses_what_does_not_fit():
    torch.cuda.set_device(0)
    lib = _lib()
    c = _case([130, 64], Hq=8, Hkv=2, D=128, P=16, split=128, seed=3)
    c["max_splits"] = STATIC_FLOATS // (c["n"] * c["Hq"] * (c["D"] + 2)) + 1
    rc, out = _run(lib, c, static=True)
    assert rc == ERR_SCRATCH
    assert float(out.float().abs().max()) == 0.0          # nothing was launched
