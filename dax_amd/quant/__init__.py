from .qscheme import per_channel_symmetric, per_tensor_symmetric, per_token_symmetric  # noqa: F401
