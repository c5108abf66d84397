"""Command-line programs: ``python -m halite_amd.cli.generate`` and
``python -m halite_amd.cli.make_random_model`` (``bin/`` holds thin launchers)."""
