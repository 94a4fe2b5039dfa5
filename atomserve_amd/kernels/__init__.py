"""Python side of the HIP kernels: building (`build`), loading (`lib`) and one
checked wrapper per kernel (`ops`)."""
