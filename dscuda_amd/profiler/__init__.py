"""Standalone profiler programs (C++, built into ``build/``) and the rocprofv3 capture / extraction driver."""
