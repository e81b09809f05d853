"""MI355X (gfx950) backend for the nanolab-GPT training-step op set of ojas.

`ojas_amd.backend.MiBackend` mirrors the reference's `Backend` trait over the
C ABI of `libojas_mi355x.so` (declared in include/ojas_mi355x.h).
"""
