"""MI355X-native batched Doom software renderer + observation pipeline (GraDOOM hot path).

The directory name is not a Python identifier; ``__graft_entry__.load_package()``
registers it under the module name ``gradoom_amd``.
"""

__version__ = "0.1.0"
