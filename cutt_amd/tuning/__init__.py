"""Tools to re-fit the planner's cost model on a GPU: collect.py times every candidate plan of a set
of random tensors with cuttPlanMeasure, fit.py turns those timings into the correction tables of
cutt_amd/csrc/model_fit.inc.  Not needed to use the library."""
