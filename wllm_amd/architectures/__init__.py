"""Architectures: each module turns its typed configuration into a ModelPlan
and registers itself under the names config.json may carry."""
from wllm_amd.architectures import duvozen  # noqa: F401  (registers Duvozen)
from wllm_amd.architectures import gemma  # noqa: F401  (registers GemmaForCausalLM)
from wllm_amd.architectures import lefisun  # noqa: F401  (registers Lefisun)
from wllm_amd.architectures import tasosun  # noqa: F401  (registers Tasosun)
from wllm_amd.architectures import tokuvik  # noqa: F401  (registers Tokuvik)
from wllm_amd.architectures.duvozen_config import DuvozenConfig  # noqa: F401
from wllm_amd.architectures.gemma_config import GemmaConfig  # noqa: F401
from wllm_amd.architectures.lefisun_config import LefisunConfig  # noqa: F401
from wllm_amd.architectures.tasosun_config import TasosunConfig  # noqa: F401
from wllm_amd.architectures.tokuvik_config import TokuvikConfig  # noqa: F401
