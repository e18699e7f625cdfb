from recflex_amd.schedules import OneHotMultiBlockSchedule, OneHotMultiBlockParams  # noqa: F401
