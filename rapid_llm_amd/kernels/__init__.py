"""Hand-written HIP kernels for gfx950 and their Python call wrappers.

``ops`` holds one function per kernel; each checks on the host that operand shapes match
what the kernel and its grid assume before anything is launched.
"""
