"""Literal inputs that the reference's own tests use (values only; no reference code).

Sources: tests/backend/cpu/ops_tests.cpp:328-337 (attention weights and input, shared with
autodiff_tests.cpp:273-282, tests/backend/cuda/ops_tests.cu:343-351, autodiff_tests.cu:373-382) and
tests/backend/cpu/autodiff_tests.cpp:234-239 (feed-forward fixture).
"""
import numpy as np

f32 = np.float32

ATTN_WQ = np.array([0.3, -0.1, 0.2, 0.05, 0.1, 0.4, -0.2, 0.15, -0.3, 0.2, 0.1, -0.05, 0.2, -0.1, 0.3, 0.1], f32).reshape(4, 4)
ATTN_WK = np.array([0.1, 0.2, -0.1, 0.3, -0.2, 0.1, 0.4, -0.1, 0.3, -0.3, 0.1, 0.2, -0.1, 0.2, -0.2, 0.1], f32).reshape(4, 4)
ATTN_WV = np.array([0.2, 0.1, -0.1, 0.3, 0.1, -0.2, 0.3, 0.1, -0.1, 0.3, 0.2, -0.1, 0.3, 0.1, -0.2, 0.2], f32).reshape(4, 4)
ATTN_WOUT = np.array([0.1, -0.1, 0.2, 0.1, 0.2, 0.1, -0.1, 0.2, -0.1, 0.2, 0.1, -0.1, 0.1, 0.2, -0.1, 0.2], f32).reshape(4, 4)
ATTN_INPUT = np.array([0.1, -0.2, 0.3, 0.4, -0.5, 0.6, 0.2, -0.1, 0.3, 0.2, -0.4, 0.5], f32).reshape(1, 3, 4)
ATTN_HEADS = 2

FF_INPUT = np.array([0.3, -0.6, 0.2, -0.4, 0.5, 0.1], f32).reshape(1, 2, 3)
FF_W1 = np.array([0.2, -0.1, 0.3, 0.1, -0.2, 0.4, 0.1, -0.3, 0.3, 0.2, -0.1, 0.2], f32).reshape(3, 4)
FF_B1 = np.array([0.1, -0.1, 0.05, 0.0], f32)
FF_W2 = np.array([0.1, -0.2, 0.3, 0.2, 0.1, -0.1, -0.3, 0.2, 0.1, 0.1, -0.1, 0.2], f32).reshape(4, 3)
FF_B2 = np.array([0.05, -0.05, 0.1], f32)
FF_GRAD = np.array([1.0, -0.5, 0.3, -0.2, 0.7, -0.4], f32).reshape(1, 2, 3)
