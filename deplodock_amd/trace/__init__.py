"""Tracers: ``nn.Module`` → frontend ``Graph``."""
