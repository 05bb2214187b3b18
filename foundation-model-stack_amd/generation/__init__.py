from .loop import default_engine, generate, generate_requests, logits, plan_batches
from .padding import pad_input_ids, trim_prefix, truncate_after_eos

__all__ = ["default_engine", "generate", "generate_requests", "logits", "pad_input_ids", "plan_batches", "trim_prefix", "truncate_after_eos"]
