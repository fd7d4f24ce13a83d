"""The reference's model zoo (torkit3d/models) on the ops of this package: PointNet,
DGCNN and PointNet++ (single-scale grouping) for classification, PointNet++ for
segmentation. Constructor arguments, sub-module names (checkpoints load unchanged),
inputs and output dictionaries are the reference's."""
