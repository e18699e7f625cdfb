from recflex_amd.schedules import OneBlockMultiSampleSchedule, OneBlockMultiSampleParams  # noqa: F401
