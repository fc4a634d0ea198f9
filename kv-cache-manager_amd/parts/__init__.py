"""Parts of a model.  Importing this package registers the built-in kinds."""
from . import llama_parts  # noqa: F401
from . import chain_norm_parts  # noqa: F401
from . import recurrent_parts  # noqa: F401
from . import conv_attention_parts  # noqa: F401
from . import side_by_side_parts  # noqa: F401
from . import gated_attention_parts  # noqa: F401
from . import routed_parts  # noqa: F401
from . import post_norm_parts  # noqa: F401
