"""The packing of a step's small arrays into one buffer (on the CPU: the same views, no page-locked memory)."""
import numpy as np
import torch

from wllm_amd.kernels.staging import pack_int32, pack_words


def test_int32_arrays_come_back_in_order_with_their_shapes():
    a = np.arange(6, dtype=np.int32).reshape(2, 3)
    b = np.zeros(0, dtype=np.int32)
    c = np.array([7, -1], dtype=np.int32)
    va, vb, vc = pack_int32([a, b, c], "cpu")
    assert va.dtype == torch.int32 and va.tolist() == a.tolist()
    assert vb.numel() == 0 and vc.tolist() == [7, -1]
    assert pack_int32([], "cpu") == []


def test_words_keep_their_kinds():
    keys = np.array([[2 ** 40 + 3, 5], [-7, 2 ** 62]], dtype=np.int64)
    table = np.array([[0.7, 40, 0.95, 0.0, 1.3]], dtype=np.float32)
    ids = np.array([3, 1, 4], dtype=np.int32)
    k, t, i = pack_words([keys, table, ids], "cpu")
    assert k.dtype == torch.int64 and k.tolist() == keys.tolist()
    assert t.dtype == torch.float32 and torch.equal(t, torch.from_numpy(table))
    assert i.dtype == torch.int32 and i.tolist() == [3, 1, 4]
