"""Latency sweeps over the shapes of the reference's benchmark scripts (benchmark/*.py), timed the
way those scripts time them: one pair of GPU events per call, median and 20 % / 80 % quantiles."""
