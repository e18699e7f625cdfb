"""Schedule templates under the module paths the reference's scripts import them from
(``examples/schedules/*.py`` of the reference); the implementations live in
``recflex_amd.schedules``."""

from recflex_amd.schedules import *  # noqa: F401,F403
