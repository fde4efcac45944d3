"""Hand-written gfx950 kernels: ``library`` builds and loads them, ``ops`` calls them."""
