from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
from . import lomozen  # noqa: F401  (registers Lomozen)
from . import dumazen  # noqa: F401  (registers Dumazen)
from . import bozisun  # noqa: F401  (registers Bozisun)
