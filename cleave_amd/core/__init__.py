"""Errors, settings, session and target: the layer everything else may import."""

from .errors import *  # noqa: F401,F403
from .errors import CleaveError  # noqa: F401
from .session import Session, active_session, current_session  # noqa: F401
from .settings import Settings  # noqa: F401
from .target import Target, current_target, default_target  # noqa: F401
