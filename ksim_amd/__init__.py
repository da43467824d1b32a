"""ksim_amd — MI355X-native rollout hot path behind ksim's engine / term / PPO interfaces."""
__version__ = "0.1.0"
