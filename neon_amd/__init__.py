"""MI355X-native implementation of neon's op-tree tensor path (backend ``hip``)."""
__version__ = "0.1.0"


class NervanaObject(object):
    """Holder of the process-wide backend handle (reference neon/__init__.py)."""
    be = None
