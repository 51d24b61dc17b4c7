from dataclasses import dataclass
from typing import Optional, Sequence


@dataclass
class MoBAConfig:
    """The reference config (moba/config.py:4-7) plus one optional field.

    full_attention_layers: indices of decoder layers (negative = counted from the last) that
    use full causal attention instead of MoBA -- the layer-wise hybrid of the technical report,
    for which the reference code has no switch.  None keeps the reference behaviour: every
    layer uses MoBA.
    """

    moba_chunk_size: int
    moba_topk: int
    full_attention_layers: Optional[Sequence[int]] = None

    def is_full_attention_layer(self, layer_idx, num_layers) -> bool:
        if not self.full_attention_layers or layer_idx is None:
            return False
        for i in self.full_attention_layers:
            if i == layer_idx or (i < 0 and num_layers is not None and num_layers + i == layer_idx):
                return True
        return False
