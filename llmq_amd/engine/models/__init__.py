"""Model registry: spec family → model class."""

from llmq_amd.engine.models.kakovik import KakovikLM
from llmq_amd.engine.models.kosalorn import KosalornLM
from llmq_amd.engine.models.llama import CausalLM
from llmq_amd.engine.models.muvetar import MuvetarLM
from llmq_amd.engine.models.tefudra import TefudraLM

MODEL_CLASSES = {
    "llama": CausalLM,
    "qwen2": CausalLM,
    "gemma2": CausalLM,
    "mistral": CausalLM,
    "kakovik": KakovikLM,
    "kosalorn": KosalornLM,
    "muvetar": MuvetarLM,
    "tefudra": TefudraLM,
}


def model_class_for(spec):
    try:
        return MODEL_CLASSES[spec.family]
    except KeyError:
        raise ValueError(f"no model class registered for family {spec.family!r}") from None


__all__ = ["CausalLM", "KakovikLM", "KosalornLM", "MuvetarLM", "TefudraLM", "MODEL_CLASSES", "model_class_for"]
