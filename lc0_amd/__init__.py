"""MI355X-native neural-network backend for lc0 (Python front end of the C ABI)."""
from .backend import (BackendError, InputPlane, Network, NetworkCapabilities,  # noqa: F401
                      NetworkComputation, library_path, load_library)
