from .convert_weights import convert_state_dict, converted_key  # noqa: F401
