from . import llama    # noqa: F401  (registers LlamaForCausalLM)
from . import suripel    # noqa: F401  (registers Suripel)
from . import sugosun    # noqa: F401  (registers Sugosun)
from . import dinasun    # noqa: F401  (registers Dinasun)
