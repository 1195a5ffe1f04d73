import sys

from tensorline_amd.cli import main

sys.exit(main())
