"""Random tensors and dropout on the emulator-backed host path."""
import nabla_amd as nb

import random_cases


def test_streams_match_the_generator(emulator):
    random_cases.check_streams_match_the_generator(nb)


def test_statistics(emulator):
    random_cases.check_statistics(nb)


def test_dropout_mask_reuse_and_reproducibility(emulator):
    random_cases.check_dropout(nb)


def test_training_mode_encoder_layer_with_default_arguments(emulator):
    random_cases.check_training_mode_encoder_layer(nb)
