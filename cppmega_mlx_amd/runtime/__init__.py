"""Runtime policy helpers (kernel-path selection and the dispatch log)."""
