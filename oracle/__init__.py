"""CPU checker for the kten-hip hot path. Test infrastructure only: the library under
kten_amd/ never imports this package."""
