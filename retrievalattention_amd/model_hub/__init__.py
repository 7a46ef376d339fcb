from .llama import LlamaModel, LlamaShape
