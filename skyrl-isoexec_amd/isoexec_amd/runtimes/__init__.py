"""Caller-side protocol of the token-logprob path: how trainer and engine reach the kernels."""
