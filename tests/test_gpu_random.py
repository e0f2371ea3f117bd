"""Random tensors and dropout on the GPU: the device generator against its numpy restatement,
element by element, and the same dropout / encoder-layer cases as the host test."""
import ctypes as C

import numpy as np
import pytest
import torch

import nabla_amd as nb

import random_cases

pytestmark = pytest.mark.gpu


def test_streams_match_the_generator(hip):
    random_cases.check_streams_match_the_generator(nb)


def test_statistics(hip):
    random_cases.check_statistics(nb)


def test_dropout_mask_reuse_and_reproducibility(hip):
    random_cases.check_dropout(nb)


def test_training_mode_encoder_layer_with_default_arguments(hip):
    random_cases.check_training_mode_encoder_layer(nb)


@pytest.mark.parametrize("n", [1, 3, 4, 1023, 70001])
def test_random_through_the_c_abi(hip, n):
    """nbk_random for every mode and a ragged length, state in device memory; nbk_rng_advance
    moves on to the next run."""
    from nabla_amd.backend import lib
    from oracle import philox
    L = lib.load()
    seed = 0x1234_5678_9ABC
    state = torch.tensor([seed, 41], dtype=torch.int64, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.full((n,), float("nan"), device="cuda")
    lib.check(L.nbk_random(out.data_ptr(), 0, n, 0, -1.0, 1.0, state.data_ptr(), 7, stream))
    np.testing.assert_array_equal(out.cpu().numpy(), philox.uniform(n, -1.0, 1.0, seed, 41, 7))
    lib.check(L.nbk_rng_advance(state.data_ptr(), stream))
    assert state.cpu().tolist() == [seed, 42]
    lib.check(L.nbk_random(out.data_ptr(), 0, n, 1, 0.0, 1.0, state.data_ptr(), 0, stream))
    np.testing.assert_allclose(out.cpu().numpy(), philox.normal(n, 0.0, 1.0, seed, 42, 0), rtol=2e-5, atol=2e-6)
    mask = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
    lib.check(L.nbk_random(mask.data_ptr(), 5, n, 2, 0.25, 0.0, state.data_ptr(), 2, stream))
    np.testing.assert_array_equal(mask.cpu().numpy().astype(bool), philox.keep_mask(n, 0.25, seed, 42, 2))
    assert L.nbk_random(mask.data_ptr(), 5, n, 0, 0.0, 1.0, state.data_ptr(), 0, stream) != 0  # uniform bytes


def test_dropout_inside_a_replayed_graph_draws_new_masks(hip):
    """A compiled step that is replayed as a recorded launch sequence still draws a new mask on
    every call: the generator state is device memory that the sequence itself advances."""
    from nabla_amd.nn import functional as F
    x = nb.Tensor.constant(np.ones((64, 128), np.float32))
    w = nb.Tensor.constant(np.ones((128, 32), np.float32))
    step = nb.compile(lambda t, w: F.dropout(t, 0.5) @ w)
    nb.set_seed(3)
    before = hip.graph_replays
    outs = []
    for _ in range(6):
        y = step(x, w)
        outs.append(y.numpy().copy())
        del y
    if hip.use_graphs:  # (NBK_GRAPHS=0: plain launches, the values are checked all the same)
        assert hip.graph_replays > before
    for a, b in zip(outs, outs[1:]):
        assert not np.array_equal(a, b)
    nb.set_seed(3)
    for want in outs:
        y = step(x, w)
        np.testing.assert_array_equal(y.numpy(), want)
        del y
