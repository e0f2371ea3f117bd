from .init import he_normal, manual_seed, normal, xavier_normal
from .layers import (dropout, embedding, gelu, layer_norm, linear, relu,
                     scaled_dot_product_attention, softmax)
from .losses import _one_hot, cross_entropy_loss, mse_loss
