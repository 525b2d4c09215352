"""fp32 form of the ADKV recurrence (the reference's train / eval arithmetic) on gfx950."""
from .train_model import ADKVTrainModel, adkv_chunk_forward, quant_f32  # noqa: F401
