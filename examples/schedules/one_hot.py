from recflex_amd.schedules import OneHotSchedule, OneHotParams  # noqa: F401
