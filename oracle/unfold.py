"""Integer index maps of the reference's unfold2D (im2col family).

Restates litenn/core/op/unfold2D.py:85-137 together with the gid -> multi-index
decomposition of litenn/core/CLKernelHelper.py:91-132 (last axis fastest).
Test infrastructure only.

An "index map" is an int64 array with one entry per element of the unfolded
matrix, in the row-major order the reference writes it (output element gid
reads flat input element map[gid]); -1 marks an element the reference sets to
zero (padding or, for the transposed map, a stride hole).
"""
import numpy as np

_SYMS = 'NCHWJI'


def _decompose(sshape, dims):
    """gid -> {symbol: index array}, following CLKernelHelper.py:91-132:
    the flat id is peeled from the last symbol to the first with % and /,
    so the output is plain row-major in the order of the symbol string.
    Returns (logical 2-D/.. shape, dict of index arrays of length size)."""
    sshape = sshape.upper()
    order = [c for c in sshape if c != '_']
    if sorted(order) != sorted(set(order)) or any(c not in _SYMS for c in order):
        raise ValueError(f'bad sshape {sshape}')
    sizes = [dims[c] for c in order]
    total = int(np.prod(sizes, dtype=np.int64))
    gid = np.arange(total, dtype=np.int64)
    idx = {}
    for c, s in zip(reversed(order), reversed(sizes)):
        idx[c] = gid % s
        gid = gid // s
    for c in _SYMS:
        idx.setdefault(c, np.zeros(total, np.int64))
    shape = [1]
    for c in sshape:
        if c == '_':
            shape.append(1)
        else:
            shape[-1] *= dims[c]
    return tuple(shape), idx


def unfold_index_map(N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE,
                     sshape='CJI_NHW'):
    """Non-transposed unfold (unfold2D.py:85-111).

    Output symbols: N batch, C channel, H/W *output* row/col, J/I kernel
    row/col.  ih = -PADT + j*DIL + h*STRIDE, iw = -PADL + i*DIL + w*STRIDE;
    element = X[n, c, ih, iw] when 0 <= ih < H and 0 <= iw < W, else 0.
    'CJI_NHW' is the reference's im2col, 'NHW_CJI' its im2row
    (conv2D.py:71-72).
    """
    shape, ix = _decompose(sshape, dict(N=N, C=C, H=OH, W=OW, J=KH, I=KW))
    ih = -PADT + ix['J'] * DILATION + ix['H'] * STRIDE
    iw = -PADL + ix['I'] * DILATION + ix['W'] * STRIDE
    ok = (ih >= 0) & (ih < H) & (iw >= 0) & (iw < W)
    flat = ((ix['N'] * C + ix['C']) * H + ih) * W + iw
    return shape, np.where(ok, flat, -1)


def unfold_T_index_map(N, C, H, W, OH, OW, KH, KW, PADL, PADT, DILATION, STRIDE,
                       sshape='NHW_CJI'):
    """Transposed unfold (unfold2D.py:113-137), as used for dX
    (conv2D.py:73: called with C=out channels, H/W = dY rows/cols,
    OH/OW = dX rows/cols).

    Output symbols H/W run over the *dX* grid (sizes OH, OW of the call);
    the source is dY[N, C, H, W].  For output position (h, w) and tap (j, i):
    sh = (PADT + h - j*DIL) / STRIDE is accepted iff it is an exact integer
    solution of h == -PADT + j*DIL + sh*STRIDE with 0 <= sh < H (same for w).
    """
    shape, ix = _decompose(sshape, dict(N=N, C=C, H=OH, W=OW, J=KH, I=KW))
    nh = PADT + ix['H'] - ix['J'] * DILATION
    nw = PADL + ix['W'] - ix['I'] * DILATION
    sh = np.floor_divide(nh, STRIDE)
    sw = np.floor_divide(nw, STRIDE)
    ok = ((nh >= 0) & (sh * STRIDE == nh) & (sh < H) &
          (nw >= 0) & (sw * STRIDE == nw) & (sw < W))
    flat = ((ix['N'] * C + ix['C']) * H + sh) * W + sw
    return shape, np.where(ok, flat, -1)


def apply_index_map(x, shape, imap):
    """Materialise the unfolded matrix from flat input x and an index map."""
    flat = np.asarray(x).reshape(-1)
    out = np.where(imap >= 0, flat[np.maximum(imap, 0)], flat.dtype.type(0))
    return out.reshape(shape)
