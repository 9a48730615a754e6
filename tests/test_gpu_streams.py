"""The measurement kernels behind `bench.py --stream-ceilings`: synthetic streams that the data kernels are
compared with.  They take no part in dispatch / combine, but a ceiling is only worth quoting if the stream
moves the bytes it claims to: every kind is checked against numpy on a small geometry (padding around the
destination stays untouched, so nothing is written out of bounds)."""
import numpy as np
import pytest
import torch

from mooncake_amd import _lib
from tests.gpu_util import announce

pytestmark = pytest.mark.gpu

PRIME = 2654435761


def _stream():
    return int(torch.cuda.current_stream().cuda_stream)


def _rows_permutation(n_rows_out_times_8, regions, used):
    j = np.arange(n_rows_out_times_8, dtype=np.uint64)
    p = (j * np.uint64(PRIME)) % np.uint64(regions * used)
    return (p % np.uint64(regions)).astype(np.int64), (p // np.uint64(regions)).astype(np.int64)


@pytest.mark.parametrize("kind", [0, 1, 2, 3, 4, 5])
def test_sequential_streams(gpu_device, kind):
    announce(f"stream kind {kind}")
    lib = _lib.lib()
    n = 3 * 256 + 40                                   # 16-byte units, not a whole number of blocks
    gen = torch.Generator().manual_seed(kind)
    src = torch.randint(0, 2 ** 31 - 1, (8 * n * 4,), generator=gen, dtype=torch.int32)
    pad = 64
    dst = torch.full((8 * n * 4 + 2 * pad,), -7, dtype=torch.int32)
    d_src, d_dst = src.cuda(), dst.cuda()
    _lib.check(lib.mc_ep_debug_stream(kind, d_dst.data_ptr() + pad * 4, d_src.data_ptr(), n * 16, _stream()))
    torch.cuda.synchronize()
    got = d_dst.cpu().numpy()
    s = src.numpy().view(np.uint32).reshape(-1, 4)
    body = got[pad:-pad].view(np.uint32).reshape(-1, 4)
    assert (got[:pad] == -7).all() and (got[-pad:] == -7).all()
    if kind == 0:
        want, rows = s[:n], n
    elif kind == 1:
        want, rows = None, 0                           # reads only
    elif kind == 2:
        want = np.stack([np.arange(n, dtype=np.uint32), np.full(n, 1, np.uint32), np.full(n, 2, np.uint32),
                         np.full(n, 3, np.uint32)], axis=1)
        rows = n
    elif kind == 3:
        h = src.numpy().view(np.uint32).reshape(-1, 2)[:n]
        want = np.stack([h[:, 0], h[:, 1], h[:, 0] ^ h[:, 1], h[:, 0] + h[:, 1]], axis=1)
        rows = n
    elif kind == 4:
        want = s[:n].copy()
        for k in range(1, 8):
            want ^= s[k * n:(k + 1) * n]
        rows = n
    else:
        o = s[0:2 * n:2] ^ s[1:2 * n:2]
        want = np.concatenate([o] * 8)
        rows = 8 * n
    if want is not None:
        assert np.array_equal(body[:rows], want)
    assert (body[rows:].view(np.int32) == -7).all()


def test_gather_of_scattered_rows(gpu_device):
    announce("gather rows")
    lib = _lib.lib()
    row_bytes, out_rows, regions, region_rows, used = 2048, 24, 12, 20, 16     # 192 source rows, each read once
    units = row_bytes // 4
    gen = torch.Generator().manual_seed(3)
    src = torch.randint(0, 2 ** 31 - 1, (regions * region_rows * units,), generator=gen, dtype=torch.int32)
    pad = 256
    dst = torch.full((out_rows * units + 2 * pad,), -7, dtype=torch.int32)
    d_src, d_dst = src.cuda(), dst.cuda()
    _lib.check(lib.mc_ep_debug_gather_rows(d_dst.data_ptr() + pad * 4, d_src.data_ptr(), row_bytes, out_rows, regions,
                                           region_rows, used, _stream()))
    torch.cuda.synchronize()
    got = d_dst.cpu().numpy()
    assert (got[:pad] == -7).all() and (got[-pad:] == -7).all()
    s = src.numpy().reshape(regions, region_rows, units)
    region, rr = _rows_permutation(out_rows * 8, regions, used)
    assert len(set(zip(region.tolist(), rr.tolist()))) == out_rows * 8 and rr.max() < used
    want = np.zeros((out_rows, units), dtype=np.int32)
    for ro in range(out_rows):
        for k in range(8):
            want[ro] ^= s[region[ro * 8 + k], rr[ro * 8 + k]]
    assert np.array_equal(got[pad:-pad].reshape(out_rows, units), want)


def test_scatter_to_scattered_rows(gpu_device):
    announce("scatter rows")
    lib = _lib.lib()
    row_bytes, in_rows, regions, region_rows, used = 1024, 20, 8, 24, 20       # 160 destination rows, each written once
    units = row_bytes // 4
    gen = torch.Generator().manual_seed(4)
    src = torch.randint(0, 2 ** 31 - 1, (in_rows * 2 * units,), generator=gen, dtype=torch.int32)
    pad = 256
    dst = torch.full((regions * region_rows * units + 2 * pad,), -7, dtype=torch.int32)
    d_src, d_dst = src.cuda(), dst.cuda()
    _lib.check(lib.mc_ep_debug_scatter_rows(d_dst.data_ptr() + pad * 4, d_src.data_ptr(), row_bytes, in_rows, regions,
                                            region_rows, used, _stream()))
    torch.cuda.synchronize()
    got = d_dst.cpu().numpy()
    assert (got[:pad] == -7).all() and (got[-pad:] == -7).all()
    body = got[pad:-pad].reshape(regions, region_rows, units)
    # a source row is 2 * row_bytes; consecutive 16-byte units are folded pairwise
    s = src.numpy().reshape(in_rows, units // 4, 2, 4)
    folded = (s[:, :, 0, :] ^ s[:, :, 1, :]).reshape(in_rows, units)
    region, rr = _rows_permutation(in_rows * 8, regions, used)
    want = np.full((regions, region_rows, units), -7, dtype=np.int32)
    for ri in range(in_rows):
        for k in range(8):
            want[region[ri * 8 + k], rr[ri * 8 + k]] = folded[ri]
    assert np.array_equal(body, want)


def test_stream_entry_points_reject_what_their_kernels_assume_away(gpu_device):
    announce("stream argument checks")
    lib = _lib.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p, st = buf.data_ptr(), _stream()
    assert lib.mc_ep_debug_gather_rows(p, p, 1000, 4, 2, 4, 2, st) != 0        # rows are whole waves: 1024-byte multiples
    assert lib.mc_ep_debug_gather_rows(p, p, 1024, 4, 2, 4, 8, st) != 0        # more rows used than a region holds
    assert lib.mc_ep_debug_scatter_rows(p, p, 1024, 4, 0, 4, 2, st) != 0
    assert lib.mc_ep_debug_stream(9, p, p, 1024, st) != 0
    assert lib.mc_ep_debug_stream(0, p, p, 1000, st) != 0
