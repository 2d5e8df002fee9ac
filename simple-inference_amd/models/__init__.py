from . import llama  # noqa: F401  (registers LlamaForCausalLM)
from . import feduzen  # noqa: F401  (registers Feduzen)
from . import mogisun  # noqa: F401  (registers Mogisun)
from . import famepel  # noqa: F401  (registers Famepel)
