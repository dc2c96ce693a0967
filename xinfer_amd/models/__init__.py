from . import debusun, lilalorn, mufenex, qwen3, vuzazen  # noqa: F401  (register the architectures)
from .registry import (ModelFamily, config_from_dict, family_of, load_config,
                       register_architecture, registered_architectures)
