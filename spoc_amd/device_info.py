"""`python -m spoc_amd.device_info`: the reference's sarek-device-info tool (tools/device_info.ml) for the
devices of this backend; exit status 1 when there is none, as there."""
import sys

from . import hip


def main():
    text, count = hip.device_report()
    sys.stdout.write(text)
    return 0 if count > 0 else 1


if __name__ == "__main__":
    sys.exit(main())
