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
* gemm.*                    pinned: linear_expected, round_to, torch_path_linear,
                            softfp8_linear_expected and torch_path_softfp8_weight
                            against float64 textbook products, closed forms
                            (alpha = 0, identity, one-hot), double-rounding known
                            answers, power-of-two scales exact, and the shipped
                            torch helper (tests/test_oracle_gemm.py); layout_c_of
                            against the reference's closed form.  The reference's
                            own expected values come from a closed-source BLAS
                            that its scripts only compare to within |diff| <= 0.1:
                            bit-level parity with that BLAS is "parity unpinned"
* router.*                  pinned (brute-force ranking, special cases, library
                            top-k on rows without ties, grouped selection with
                            and without bias by brute force, one group == plain)
* align.*                   pinned (invariants + brute force on the 64-entry
                            example input the reference holds)
* moe.*                     pinned (float64 brute force on tiny shapes; the dense
                            masked-sum torch path through its grouped / sigmoid /
                            bias / expert-map branches against the router oracle
                            and the sparse statement, with a dropped-pick control)
* selector.*                pinned (known-answer rows through multi-row tables with
                            decoys, duplicate keys and short rows)
"""
