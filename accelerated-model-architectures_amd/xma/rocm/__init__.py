from .loader import LIBRARY_PATH, RocmLibraryError, get_library, is_library_built
