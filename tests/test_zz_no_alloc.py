"""The entry point that allocates nothing: ``gs_attention_decode_static``, called through ctypes.

Its partial results lie in a static device array instead of a workspace the caller brings; its output must
equal, bit for bit, that of ``gs_attention_decode`` with a caller's workspace (the kernels are the same), on two
calls in a row of which the second is smaller, so that what the first call left in the array is in the way.
A call that needs more than the array holds is refused before anything is launched.
"""
import ctypes
import math
from ctypes import c_float, c_int, c_void_p

import pytest
import torch

import plain_lfm2 as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
STATIC_FLOATS = 1 << 20


def _case(seed, lens, nh, nkv, d, ps):
    g = torch.Generator().manual_seed(seed)
    nseq = len(lens)
    nblk = [-(-n // ps) for n in lens]
    total = sum(nblk)
    perm = torch.randperm(total + 2, generator=g)[:total] + 1
    kc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    vc = torch.randn(total + 3, nkv, ps, d, generator=g).bfloat16()
    table = torch.zeros(nseq, max(nblk), dtype=torch.int32)
    q = torch.randn(nseq, nh * d, generator=g).bfloat16()
    want, at = [], 0
    for i, n in enumerate(lens):
        pages = perm[at:at + nblk[i]]
        at += nblk[i]
        table[i, :nblk[i]] = pages.to(torch.int32)
        k = kc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n]
        v = vc[pages].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:n]
        want.append(P.causal_attention(q[i].double().reshape(1, nh, d), k.double(), v.double(), 0).reshape(-1))
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    return dict(q=q.to(DEV), kc=kc.to(DEV), vc=vc.to(DEV), table=table.to(DEV), positions=positions.to(DEV),
                want=torch.stack(want), nseq=nseq)


def _call(lib, name, c, nh, nkv, d, ps, nsplit, workspace=None):
    out = torch.full((c["nseq"], nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    p = lambda t: c_void_p(t.data_ptr())
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [p(c["q"]), c_int(nh * d), p(c["kc"]), p(c["vc"]), p(c["positions"]), p(c["table"]),
            c_int(c["table"].shape[1]), c_int(ps), c_int(0), c_float(1.0 / math.sqrt(d)), p(out), c_int(0)]
    if workspace is not None:
        args.append(p(workspace))
    args += [c_int(c["nseq"]), c_int(nh), c_int(nkv), c_int(d), c_int(nsplit), stream]
    fn = getattr(lib, name)
    fn.restype = c_int
    rc = fn(*args)
    torch.cuda.synchronize()
    return rc, out


def test_static_workspace_gives_what_the_callers_workspace_gives():
    from gesso_amd.kernels import ops
    lib = ops.lib()
    lib.gs_attention_decode_workspace.restype = ctypes.c_long
    nh, nkv, d, ps = 8, 2, 64, 16
    # the second call is smaller in every way: fewer sequences, fewer keys, fewer splits
    for seed, lens, nsplit in ((1, [700, 64, 1500, 129, 1, 300], 8), (2, [65, 400], 3)):
        c = _case(seed, lens, nh, nkv, d, ps)
        floats = lib.gs_attention_decode_workspace(c_int(c["nseq"]), c_int(nh), c_int(nkv), c_int(d), c_int(nsplit))
        assert 0 < floats <= STATIC_FLOATS
        ws = torch.full((floats,), float("nan"), dtype=torch.float32, device=DEV)
        rc, ref = _call(lib, "gs_attention_decode", c, nh, nkv, d, ps, nsplit, workspace=ws)
        assert rc == 0, lib.gs_last_error().decode()
        rc, got = _call(lib, "gs_attention_decode_static", c, nh, nkv, d, ps, nsplit)
        assert rc == 0, lib.gs_last_error().decode()
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), "static and caller's workspace differ"
        diff = float((got.double().cpu() - c["want"]).abs().max())
        assert diff <= 1e-2 * max(1.0, float(c["want"].abs().max())), diff


def test_static_workspace_refuses_more_than_it_holds():
    from gesso_amd.kernels import ops
    lib = ops.lib()
    nh, nkv, d, ps = 32, 8, 128, 16
    c = _case(3, [40] * 16, nh, nkv, d, ps)              # 16 x 32 x 64 x 130 floats: above the static array
    rc, out = _call(lib, "gs_attention_decode_static", c, nh, nkv, d, ps, 64)
    assert rc != 0 and "static" in lib.gs_last_error().decode()
    assert bool(torch.isnan(out.float()).all())           # nothing was launched
