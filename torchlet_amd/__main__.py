import sys

from .llm import main

sys.exit(main())
