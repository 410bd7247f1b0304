"""Registers the Narolorn decoder: the name in config.json -> its configuration class."""
from ..config.narolorn import NarolornConfig
from ..registry import register

register("architecture", "Narolorn")(NarolornConfig)
