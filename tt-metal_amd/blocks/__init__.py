"""The callers either side of the block-float GEMMs: the MLP blocks of Falcon-7B and Mistral-7B as tt-metal's model
code writes them (models/demos/falcon7b/tt/falcon_mlp.py, models/demos/mistral7b/tt/mistral_mlp.py), on this build's
tt_lib / ttnn surface."""
from .falcon_mlp import TtFalconMLP, falcon_mlp_model_config  # noqa: F401
from .mistral_mlp import TtMistralMLP, mistral_mlp_model_config  # noqa: F401
