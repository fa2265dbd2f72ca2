from .registry import (config_from_checkpoint, get_model_config, list_models,
                       register, resolve_model_class)
