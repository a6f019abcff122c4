"""MI355X-native members of the Eric model zoo.

They follow the zoo's own recipe (reference: eric/models/__init__.py:1-11): one module per
`hf_config.model_type`, a class inheriting `EricModel`, a class named exactly `ModalityProcessor`, and an
entry in `MODEL_REGISTRY`.
"""
