'''CPU oracle for the vkJAX device path. TEST INFRASTRUCTURE ONLY: imported by tests/,
by the smoke entry and by the benchmark's CPU-baseline leg; never by the shipped package.'''
