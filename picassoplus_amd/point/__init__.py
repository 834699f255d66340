"""Point-cloud modules with the API of ``picasso.point`` of the reference."""
from . import pi_modules  # noqa: F401
