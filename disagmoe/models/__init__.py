"""Expert-worker part of the reference package of the same name."""
