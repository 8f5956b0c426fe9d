"""Parts that layers are assembled from. Importing the package registers the built-in parts."""

from tinyserve_llm_amd.parts import base  # noqa: F401
from tinyserve_llm_amd.parts import (attention, block, ends, latent, linear_attention, mingru, mlp, mlstm, moe, norm, rope,  # noqa: F401
                                     side_by_side, stream, token_input)  # noqa: F401  (registration)
