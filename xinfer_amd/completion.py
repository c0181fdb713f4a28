"""`python -m xinfer_amd.completion`: the reference ships its Python example under this
module name (/root/reference/build.sh:170-175); same options as `python -m xinfer_amd`."""
import sys

from .cli import main

if __name__ == "__main__":
    sys.exit(main())
