from kvforge_amd.models import llama  # noqa: F401  (registers LlamaForCausalLM)
