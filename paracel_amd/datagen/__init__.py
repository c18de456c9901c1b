"""Seeded synthetic shards (host side) -- ctypes binding of libplr_gen.so and
the five benchmark configurations."""
from .gen import *  # noqa: F401,F403
