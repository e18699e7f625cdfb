from recflex_amd.schedules import WarpPerSampleSchedule, WarpPerSampleParams  # noqa: F401
