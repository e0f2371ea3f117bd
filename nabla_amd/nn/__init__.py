from . import finetune, functional
from .modules import (GELU, Dropout, Embedding, LayerNorm, Linear, Module, MultiHeadAttention,
                      ReLU, Sequential, TransformerEncoderLayer)
