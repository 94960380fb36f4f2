"""Code generators.  There is exactly one: :mod:`appy_amd.backends.hip`."""
