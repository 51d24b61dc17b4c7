from dataclasses import dataclass


@dataclass
class MoBAConfig:
    """Same two fields as the reference config (moba/config.py:4-7)."""

    moba_chunk_size: int
    moba_topk: int
