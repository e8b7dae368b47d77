"""MI355X-native inference engine for the Qwen2.5 dense decoder.

Import name ``cie_amd`` (see ``cie_amd.py`` at the repository root).
"""

__version__ = "0.1.0"
