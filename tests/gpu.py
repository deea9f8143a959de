"""GPU-side plumbing for the tests: numpy <-> device buffers (torch is only the allocator) and the C ABI wrappers."""
import numpy as np
import torch

from dsgx10_amd import abi, lib  # noqa: F401


def dev(a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view(np.uint8).reshape(-1)).cuda()


def empty(nbytes, fill=None):
    t = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    if fill is not None:
        t.fill_(fill)
    return t


def view(base, ptr, nbytes):
    """the bytes [ptr, ptr + nbytes) of the device buffer `base` (a pointer the library returned into it)"""
    o = int(ptr) - base.data_ptr()
    assert 0 <= o and o + nbytes <= base.numel()
    return base[o:o + nbytes]


def host(t, dtype, shape):
    torch.cuda.synchronize()
    return t.cpu().numpy().view(dtype).reshape(shape).copy()


def decode_layer(dl, x, idx, w, M, ws=None, **kw):
    """runs dsgx_moe_decode; returns (yr f32 [M][H], ys f32 [M][H], ws tensor)"""
    H = dl.host.H
    if ws is None:
        ws = empty(lib.decode_ws_bytes(dl.w), 0)
    dx, di, dw = dev(x), (None if idx is None else dev(idx)), (None if w is None else dev(w))
    yr, ys = empty(M * H * 4, 0xFF), empty(M * H * 4, 0xFF)
    kw.setdefault("up", 0)  # a named variant: a row's bits are then the same at every row count
    if kw.get("ys_in") is not None:
        ys = dev(kw.pop("ys_in"))
    else:
        kw.pop("ys_in", None)
    lib.moe_decode(dl.w, dx, di, dw, M, ws, yr, ys, **kw)
    lib.decode_status(dl.w, ws)  # (raises if a fused step gave up at its grid barrier)
    return host(yr, np.float32, (M, H)), host(ys, np.float32, (M, H)), ws


def h_of(ws, dl, M, nslots):
    """h bf16 [nslots (+1 shared, last)][M][I] out of the decode workspace"""
    I = dl.host.I
    hb = host(ws[: (abi.MAX_UNION + 1) * abi.MAX_ROWS * I * 2], np.uint16, (-1,))
    sl = list(range(nslots)) + ([abi.SH_SLOT] if dl.host.has_shared else [])
    return np.stack([hb[s * M * I:(s + 1) * M * I].reshape(M, I) for s in sl])
