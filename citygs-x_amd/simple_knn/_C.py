"""Drop-in for simple_knn._C (submodule_cityx/simple-knn/ext.cpp:15-17)."""
import ctypes as C

import torch

import gsrast_native as _n


def distCUDA2(points):
    """Mean squared distance of every point to its three nearest neighbours
    (submodule_cityx/simple-knn/spatial.cu:17-35).  points: (P,3) float32 GPU tensor."""
    if not points.is_cuda:
        raise RuntimeError("distCUDA2 needs a GPU tensor: there is no CPU path")
    if points.dtype != torch.float32:
        raise TypeError("points must be float32")
    pts = points.contiguous()
    P = pts.shape[0]
    dev = pts.device
    out = torch.zeros(P, dtype=torch.float32, device=dev)
    if P == 0:
        return out
    nbytes = _n.lib.gs_knn_workspace_bytes(P)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _n.check(_n.lib.gs_knn_dist2(P, C.c_void_p(pts.data_ptr()), C.c_void_p(out.data_ptr()),
                                     C.c_void_p(ws.data_ptr()), nbytes,
                                     C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "distCUDA2")
    return out
