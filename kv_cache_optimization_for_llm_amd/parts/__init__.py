"""Parts a layer is put together from; importing this package registers the built-in kinds."""
from . import base, linear, norm, rotary, attention, latent_attention, mlp, block, stream_ops, recurrent, composite, moe, layer_input  # noqa: F401
