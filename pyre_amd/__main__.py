import sys

from pyre_amd.cli import main

sys.exit(main())
