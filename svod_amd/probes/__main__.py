import sys

from . import build, run

if __name__ == "__main__":
    if "--build" in sys.argv[1:]:
        print("\n".join(build(verbose=True)))
    else:
        import os

        from . import BIN, PROBES

        if not all(os.path.exists(os.path.join(BIN, p)) for p in PROBES):
            build()
        run()
