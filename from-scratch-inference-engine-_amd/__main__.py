from .engine.cli import main

raise SystemExit(main())
