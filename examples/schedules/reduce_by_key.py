from recflex_amd.schedules import ReduceByKeySchedule, ReduceByKeyParams  # noqa: F401
