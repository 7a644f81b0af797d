"""Package logger; silent unless the application configures logging
(same policy as the reference's ``spikingjelly/logger.py:39-42``)."""

import logging

logger = logging.getLogger("spikingjelly_amd")
logger.addHandler(logging.NullHandler())
