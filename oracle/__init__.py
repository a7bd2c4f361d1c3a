"""CPU oracle for the native-layout GeMV / narrow-GeMM / fused-MoE path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only the tests, the smoke check and the benchmark's CPU-baseline
leg do, and there only as the checker.  Each function restates, on the CPU
with numpy / CPU torch, what the reference computes, and cites the reference
file:line it follows.  How every function is pinned (closed forms, library
routines, brute force, invariants) is listed in the function's docstring.

Parity status of the functions in this package:

* layouts.*                 pinned (closed-form view/permute held by the
                            reference's scripts + independent index loops)
* softfp8.*                 pinned (exhaustive 256-code table against the
                            library float8_e4m3fn decode; NaN codes closed form)
* gemm.*                    pinned to the textbook product; the reference's own
                            expected values come from a closed-source BLAS that
                            its scripts only compare to within |diff| <= 0.1,
                            so bit-level parity of that BLAS is unpinned
* router.*                  pinned (brute-force ranking, special cases,
                            library top-k on rows without ties)
* align.*                   pinned (invariants + brute force on the 64-entry
                            example input the reference holds)
* moe.*                     pinned (float64 brute force on tiny shapes, dense
                            masked sum == sparse gather identity)
* selector.*                pinned (known-answer rows of the reference's tables)
"""
