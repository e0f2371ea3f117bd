from . import finetune, functional, optim
from .modules import (GELU, Dropout, Embedding, LayerNorm, Linear, Module, MultiHeadAttention,
                      ReLU, Sequential, TransformerEncoderLayer)
