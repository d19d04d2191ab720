"""HIP sources of the gfx950 kernels and the driver that compiles them."""
