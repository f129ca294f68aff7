"""nnv_amd: MI355X-native star-set reachability (relax-star, relaxFactor = 1) behind NNV's API."""
