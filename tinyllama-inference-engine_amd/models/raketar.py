"""Registers the Raketar decoder: the name in config.json -> its configuration class."""
from ..config.raketar import RaketarConfig
from ..registry import register

register("architecture", "Raketar")(RaketarConfig)
