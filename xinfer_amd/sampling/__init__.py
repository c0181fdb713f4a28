from .sampler import PENALTY_CONTEXT, Sampler, Strategy, get_strategy, resolve_strategy, uniform
