from .codegen import CodeEmitter
from .schedule_base import ScheduleBase, ScheduleVars, PreprocessVars, InputStats, MetaData
