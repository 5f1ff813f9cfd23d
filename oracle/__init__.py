"""CPU oracle for the WKV time-mix recurrence.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only the test-suite, the smoke check and the benchmark's
``cpu_baseline`` leg do, and there only as the checker / the timed CPU
baseline.  The shipped operators fail loudly when the HIP library is missing
instead of falling back to anything in here.

Contents
--------
wkv56.py   restatement of the reference's pure-PyTorch WKV5/WKV6 path
           (RWKV-v5/src/module/rwkv_inner.py:10-118,
           RWKV-v6/src/module/rwkv_inner.py:10-115) plus an independent
           per-token statement and closed-form adjoints.
wkv4.py    restatement of the v4 recurrence with (aa, bb, pp) state
           (RWKV-v4neo/cuda/wkv_cuda_bf16.cu:7-158), Python/torch front-end.
wkv4_ref.c plain-C restatement of the same v4 forward/backward, built by
           oracle/Makefile into oracle/libwkv4_oracle.so.

Pinning status (what fixes each function besides its own formula)
-----------------------------------------------------------------
The reference ships no tensor-level test, golden vector or known-answer file
for this path, its CUDA sources need nvcc (absent) and its Python module
imports packages that are not installed, so nothing of the reference was
built or run.  Every function is pinned by mathematics instead; the tests
that do so are named beside each function.  No function is left unpinned.
"""
