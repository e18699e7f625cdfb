from .tuner import Tuner, TuneConfig, BasicConfig
