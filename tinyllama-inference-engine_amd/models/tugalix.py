"""Registers the Tugalix decoder: the name in config.json -> its configuration class."""
from ..config.tugalix import TugalixConfig
from ..registry import register

register("architecture", "Tugalix")(TugalixConfig)
