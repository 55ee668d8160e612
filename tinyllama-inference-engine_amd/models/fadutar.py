"""Registers the Fadutar decoder: the name in config.json -> its configuration class."""
from ..config.fadutar import FadutarConfig
from ..registry import register

register("architecture", "Fadutar")(FadutarConfig)
