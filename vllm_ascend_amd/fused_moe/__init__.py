"""Routed-experts runtime: router, token dispatch, grouped-GEMM MLP, combine."""
