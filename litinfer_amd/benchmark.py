"""placeholder"""
def main(argv=None):
    raise SystemExit("bench: not wired yet")
