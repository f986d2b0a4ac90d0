"""Python front end of the MI355X build of Mini-Caffe's forward path."""
from .base import LIB, LIB_PATH, MiniCaffeError  # noqa: F401
