"""oneshot(model, recipe): apply a recipe in place (llmquant/core/oneshot.py:6-12)."""

from __future__ import annotations


def load_pretrained(args):
    """(model, tokenizer) for a model id or local path, on args.device, in eval mode."""
    import torch
    from transformers import AutoModelForCausalLM, AutoTokenizer

    tokenizer = AutoTokenizer.from_pretrained(args.model_id)
    model = AutoModelForCausalLM.from_pretrained(args.model_id, dtype=getattr(torch, args.dtype))
    return model.to(args.device).eval(), tokenizer


def oneshot(model, recipe):
    """`model` is a loaded nn.Module, or a model id / path, in which case (model, tokenizer)
    comes back."""
    if isinstance(model, str):
        from llmquant.core.config import ModelArgs

        loaded, tokenizer = load_pretrained(ModelArgs(model_id=model))
        recipe.apply(loaded)
        return loaded, tokenizer
    recipe.apply(model)
    return model
