from kvforge_amd.models import fogorax  # noqa: F401  (registers Fogorax)
from kvforge_amd.models import rudorax  # noqa: F401  (registers Rudorax)
from kvforge_amd.models import llama  # noqa: F401  (registers LlamaForCausalLM)
from kvforge_amd.models import buzinex  # noqa: F401  (registers Buzinex)
