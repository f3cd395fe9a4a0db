"""MI355X-native recurrent fast-weight operators (SRWM and delta rule).

The directory is meant to be put on sys.path in place of the reference's extension
directories, so `from self_ref_v0 import self_ref_v0` and
`from fast_weight import fast_weight_delta` resolve to the HIP-backed operators.
"""
