"""MSCCLang algorithms shipped with the package.  Each function issues chunk operations inside an
active MSCCLProgram; `build_*` helpers in `msccl.programs.catalog` wrap them into complete programs."""
