from .loader import default_weight_loader, load_model  # noqa: F401
