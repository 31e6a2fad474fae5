"""CPU checkers for the HIP path: test infrastructure, never imported by the product package.

`oracle.lib`     ctypes bindings of liboracle.so (this repo's strict-fp32 restatement) and, when it
                 was built, of _ref/libskainet_ref.so (the reference's own C kernels).
`oracle.golden`  the reference's golden-test input generator and digest, restated.
"""
