import sys

from sprout_lm_amd.cli import main

sys.exit(main())
