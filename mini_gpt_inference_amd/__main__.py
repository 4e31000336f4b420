from .generate import main

raise SystemExit(main())
