"""``python -m isoexec_amd.debug TRACE_A TRACE_B`` compares two trace directories (see ``compare``)."""

import sys

from .compare import main

sys.exit(main())
