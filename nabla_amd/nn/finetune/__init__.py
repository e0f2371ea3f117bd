from .lora import (init_lora_adapter, lora_delta, lora_linear, merge_lora_weight,
                   unmerge_lora_weight)
