"""`eager` (CPU) lane of lattice_rans. Placeholder until the encoder lands."""


def encode(**kwargs):
    raise NotImplementedError("CPU encoder not built yet")


def decode(buffers, *, shape, dtype, threads_per_block=None, l2_prefetch=True):
    raise RuntimeError(
        "this package has no CPU decoder: lattice_rans containers are decoded by the hip lane (MI355X). "
        "Pass execution_backend='hip' on a machine with a gfx950 device.")
