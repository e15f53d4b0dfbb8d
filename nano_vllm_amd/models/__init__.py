from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
from . import nozurax  # noqa: F401  (registers Nozurax)
from . import mafarax  # noqa: F401  (registers Mafarax)
from . import kirisun  # noqa: F401  (registers Kirisun)
