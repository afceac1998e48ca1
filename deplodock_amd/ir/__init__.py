"""IR levels: frontend ops (what is computed), tile ops (how one kernel is scheduled), HipOp (source + launch)."""
