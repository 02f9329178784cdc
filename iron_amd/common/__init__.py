"""The layer under the operators: declarations, judging, testing, graphs, arena."""
