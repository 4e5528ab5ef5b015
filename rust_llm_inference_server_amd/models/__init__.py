"""Models as data (``ModelSpec``) and the architectures that ship with the package."""
from .bekunex import bekunex_spec
from .gipotar import gipotar_spec
from .lagedra import lagedra_spec
from .llama import llama_spec
from .pamolix import pamolix_spec
from .spec import LayerSpec, Model, ModelSpec, RunEntry

__all__ = ["LayerSpec", "Model", "ModelSpec", "RunEntry", "bekunex_spec", "gipotar_spec",
           "lagedra_spec", "llama_spec", "pamolix_spec"]
