"""bin_by_coordinates on MI355X.  Mirrors the reference wrapper
fastgraphcompute/extensions/bin_by_coordinates.py:11-111 (same signature,
same five return values, same ValueErrors); the tensor preprocessing and the
per-point kernel run as HIP kernels of libfgc_hip.so."""
from typing import Optional, Tuple

import torch

from .. import _lib


def bin_by_coordinates(coordinates: torch.Tensor, row_splits: torch.Tensor,
                       bin_width: Optional[torch.Tensor] = None, n_bins: Optional[torch.Tensor] = None,
                       calc_n_per_bin: bool = True, pre_normalized: bool = False,
                       name: str = "") -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Assign every point to a bin of a regular grid, per event.

    Returns (bin_indices [N, D+1] int64 with column 0 the event, flat_bin_indices
    [N] int64, n_bins [D] int64, bin_width [1] float32, n_per_bin [B] int64).
    """
    _lib.require_device(coordinates)
    L = _lib.lib()
    dev = coordinates.device
    coords = coordinates.to(torch.float32).contiguous()
    if coords.dim() != 2:
        raise ValueError("coordinates must be [n_vert, n_coords]")
    n, d = coords.shape
    if d < 1 or d > 5:
        raise ValueError("Unsupported number of binning dimensions.")
    rs = row_splits.to(device=dev, dtype=torch.int64).contiguous()
    n_rs = rs.numel()

    if bin_width is None and n_bins is None:
        raise ValueError("Either bin_width or n_bins must be provided.")
    nb_host = None
    if n_bins is not None:
        nb_t = n_bins if torch.is_tensor(n_bins) else torch.tensor(n_bins, dtype=torch.int64)
        nb_t = nb_t.to(torch.int64).cpu()
        if nb_t.dim() == 0:
            nb_t = nb_t.repeat(d)
        nb_host = [int(v) for v in nb_t.tolist()]
        if len(nb_host) != d:
            raise ValueError("bin_by_coordinates: coordinates.size(1) must be equal to nbins.size(0)")
        if not all(v > 0 for v in nb_host):
            raise ValueError("BinByCoordinates: n_bins must be greater than zero.")
    bw_host = 0.0
    if bin_width is not None:
        bw_t = bin_width if torch.is_tensor(bin_width) else torch.tensor([bin_width], dtype=torch.float32)
        if bw_t.numel() != 1:
            raise ValueError("bin_by_coordinates: bin_width must be a singleton tensor")
        bw_host = float(bw_t.to(torch.float32).reshape(-1)[0].item())
        if not bw_host > 0:
            raise ValueError("BinByCoordinates: bin_width must be greater than zero.")

    if n == 0:
        nb_out = torch.tensor(nb_host if nb_host is not None else [1] * d, dtype=torch.int64, device=dev)
        B = int(torch.prod(nb_out).item()) * max(n_rs - 1, 0)
        return (torch.empty((0, d + 1), dtype=torch.int64, device=dev), torch.empty((0,), dtype=torch.int64, device=dev),
                nb_out, torch.tensor([bw_host], dtype=torch.float32, device=dev),
                torch.zeros((B,), dtype=torch.int64, device=dev))

    geom = torch.empty(16, dtype=torch.float32, device=dev)
    status = torch.zeros(4, dtype=torch.int32, device=dev)
    ws_bytes = L.fgc_bin_geometry_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    mode = 0 if bin_width is None else 1
    nb_arr = _lib.host_i64(nb_host if nb_host is not None else [1] * d)
    with torch.cuda.device(dev):
        st = _lib.stream_ptr()
        _lib.check(L.fgc_bin_geometry_f32(_lib.ptr(coords), n, d, d, mode, nb_arr, 1 if nb_host is not None else 0,
                                          bw_host, 1 if pre_normalized else 0, _lib.ptr(geom), _lib.ptr(status),
                                          _lib.ptr(ws), ws_bytes, st))
        g = geom.cpu()  # one synchronisation: n_bins sizes the outputs, flags carry the input checks
        flags = int(g[11:12].view(torch.int32).item())
        if flags & _lib.ST_NONFINITE:
            raise ValueError(f"BinByCoordinates: input coordinates {name} contain non-finite values")
        nb_final = [int(v) for v in g[6:6 + d].view(torch.int32).tolist()]
        if flags & _lib.ST_BAD_RANGE:
            if not all(v > 0 for v in nb_final):
                raise ValueError("BinByCoordinates: n_bins must be greater than zero.")
            raise ValueError("BinByCoordinates: dmax_coords must be greater than zero.")
        B = max(n_rs - 1, 0)
        for v in nb_final:
            B *= v
        assigned = torch.empty((n, d + 1), dtype=torch.int64, device=dev)
        flat = torch.empty((n,), dtype=torch.int64, device=dev)
        nper = torch.zeros((B,), dtype=torch.int64, device=dev)
        nbf = _lib.host_i64(nb_final)
        _lib.check(L.fgc_bin_points_f32(_lib.ptr(coords), n, d, d, _lib.ptr(geom), _lib.ptr(rs), n_rs, nbf,
                                        _lib.ptr(assigned), _lib.ptr(flat),
                                        _lib.ptr(nper) if calc_n_per_bin else None, _lib.ptr(status), st))
    nb_out = torch.tensor(nb_final, dtype=torch.int64, device=dev)
    bw_out = geom[5:6].clone()
    return assigned, flat, nb_out, bw_out, nper
