"""Hook for running nengo's own test suite against this backend.

Counterpart of the reference's ``nengo_ocl/tests/__init__.py:6-17``: nengo's pytest plugin
reads the option ``nengo_simloader`` and calls the function it names to get the
``Simulator`` fixture.  With nengo installed::

    pytest --pyargs nengo -c <this package>/nengo_tests.cfg

``nengo_tests.cfg`` names this loader, the neuron types to test and the tests this backend
does not support, with the reason for each (the reference keeps that list in its
``setup.cfg:55-108``).
"""


def make_test_sim(request):
    """A Simulator factory for nengo's ``Simulator`` test fixture."""
    import nengo_ocl_amd

    def TestSimulator(net, *args, **kwargs):
        kwargs.setdefault("progress_bar", False)
        return nengo_ocl_amd.Simulator(net, *args, **kwargs)

    return TestSimulator
