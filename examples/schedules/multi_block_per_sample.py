from recflex_amd.schedules import MultiBlockPerSampleSchedule, MultiBlockPerSampleParams  # noqa: F401
