"""MI355X-native LowOHA int8 matmul path (see include/zmi_lowoha.h)."""
__version__ = "0.1.0"
