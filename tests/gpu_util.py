"""Runs a workload on the GPU through the public API (flat C ABI) with torch-owned buffers."""
import numpy as np

from hiptensor_amd import api
from hiptensor_amd import workloads as wl


def to_device(buf):
    import torch

    return torch.from_numpy(buf.view(np.uint8).copy()).cuda()


def run_gpu(handle, w, inp=None, algo=api.HIPTENSOR_ALGO_DEFAULT, pref=api.HIPTENSOR_WORKSPACE_RECOMMENDED,
            d_alias_c=False, workspace_limit=None, return_info=False):
    """Returns D as a host array of the storage type (span elements)."""
    import torch

    if inp is None:
        inp = wl.host_inputs(w)
    A, B = to_device(inp["A"]), to_device(inp["B"])
    Cd = to_device(inp["C"]) if inp["C"] is not None else None
    if d_alias_c:
        D = Cd
    else:
        D = to_device(wl.nan_buffer(w["dtype"], inp["spanD"]))
    # alignment from the pointers, the way the reference's samples and tests obtain it
    c = wl.Contraction(handle, w, algo=algo, pref=pref, workspace_limit=workspace_limit)
    ws = torch.empty(max(int(c.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    st = c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr() if Cd is not None else None, D.data_ptr(),
               ws.data_ptr() if c.workspace_bytes else None, stream)
    torch.cuda.synchronize()
    info = dict(c.info)
    c.close()
    api.check(st, "hiptensorContraction " + w["name"])
    out = D.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
    return (out, info) if return_info else out


def run_gpu_permutation(handle, w, A=None, a_shift=0, b_shift=0, return_info=False):
    """Runs one permutation workload; returns packed B as a host array of the storage type.
    a_shift / b_shift move the two device tensors off their allocation's alignment by that
    many elements.  B is pre-filled with NaN, so an element left unwritten shows."""
    import torch

    if A is None:
        A = wl.permutation_input(w)
    t = wl.NP_STORE[w["dtype"]]
    n = max(int(np.prod(w["lensB"])), 1)
    item = np.dtype(t).itemsize
    hostA = np.concatenate([np.zeros(a_shift, dtype=t), np.ascontiguousarray(A, dtype=t)])
    dA = to_device(hostA)
    dB = to_device(wl.nan_buffer(w["dtype"], n + b_shift))
    p = wl.Permutation(handle, w)
    pa, pb = dA.data_ptr() + a_shift * item, dB.data_ptr() + b_shift * item
    info = p.info(pa, pb)
    st = p.run(pa, pb, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    p.close()
    api.check(st, "hiptensorPermutation " + w["name"])
    out = dB.cpu().numpy().view(t)[b_shift:]
    return (out, info) if return_info else out
