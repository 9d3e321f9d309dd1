"""yalis_amd: a small, whole inference engine for one MI355X."""
