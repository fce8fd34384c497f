import sys

from turboserve_amd.cli import main

sys.exit(main())
