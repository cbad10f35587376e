from . import qwen2  # noqa: F401  (registers Qwen2ForCausalLM)
from . import napadra  # noqa: F401  (registers Napadra)
from . import dolidra  # noqa: F401  (registers Dolidra)
from . import bokulorn  # noqa: F401  (registers Bokulorn)
