"""Typed configurations read from config.json."""

from .reader import ConfigError, KeyReader, read_json
from .minimax_m3 import MiniMaxM3Config
from .nenotar import NenotarConfig
from .bonerax import BoneraxConfig
from .givozen import GivozenConfig
from .salipel import SalipelConfig

__all__ = ["ConfigError", "KeyReader", "read_json", "MiniMaxM3Config", "NenotarConfig", "BoneraxConfig", "GivozenConfig", "SalipelConfig"]
