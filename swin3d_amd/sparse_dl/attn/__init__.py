from .attn_coff import (IndexMode, PosEmb, PrecisionMode, SelfAttnAIOFunction, TableDims,
                        window_attention_backward, window_attention_forward)
