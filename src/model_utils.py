"""Same import path as the reference's src/model_utils.py: the cache hook lives in hqmq_amd.hf_cache.

`QuantizedCache` is the reference's fake-quantizing DynamicCache; `PackedQuantizedCache` keeps the layers
bit-packed and attends from the compressed planes (attn_implementation="hqmq_packed").
`load_model` needs the Hugging Face hub and is here for signature compatibility only.
"""
import torch

from hqmq_amd.hf_cache import ATTN_NAME, PackedQuantizedCache, QuantizedCache  # noqa: F401


def load_model(model_name: str, dtype: torch.dtype = torch.float16, device: str = "cuda"):
    """Load an HF causal LM + tokenizer (reference: src/model_utils.py:35-43). Returns (model, tokenizer)."""
    from transformers import AutoModelForCausalLM, AutoTokenizer
    tokenizer = AutoTokenizer.from_pretrained(model_name)
    model = AutoModelForCausalLM.from_pretrained(model_name, dtype=dtype, attn_implementation="eager").to(device)
    model.eval()
    return model, tokenizer
