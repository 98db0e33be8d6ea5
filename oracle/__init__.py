"""CPU oracle for the SAM ViT image-encoder hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, on the CPU, what the
reference computes on the hot path (rel-pos attention, window partition,
dynamic int8 linears, the encoder that hosts them).  It is the checker the
parity tests, the smoke run and the bench's CPU-baseline leg compare the HIP
path against.  Nothing in the product package imports it, and the product
never falls back to it.

Everything here is plain torch-on-CPU / numpy written from the formulas, one
function per reference function, each citing the reference file:line it
follows.  How each function is pinned (closed forms, brute force, library
routines, invariants) is listed in that function's module header; functions
that nothing but an import of an absent third-party package could pin say
"parity unpinned" there.
"""
