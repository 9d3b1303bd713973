"""Source folder of the ``llmserve`` package (imported through ``llmserve/__init__.py``)."""
