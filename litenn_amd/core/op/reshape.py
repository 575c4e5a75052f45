import litenn_amd.core as nc


def reshape(input_t, target_shape):
    """Zero-copy reshape: a reference tensor over the same storage
    (reshape.py:7-18).  target_shape may hold one -1."""
    info = nc.Cacheton.get(nc.info.InfoReshape, input_t.shape, tuple(int(x) for x in target_shape))
    return input_t._as_ref(info.output_shape)


def flatten(input_t):
    """reshape(x, (x.shape[0], -1))   (reshape.py:20-26)."""
    return reshape(input_t, (input_t.shape[0], -1))
