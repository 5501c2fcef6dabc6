"""Build functions of this backend for nengo objects.

Counterpart of the reference's ``nengo_ocl/builder.py`` (:11-51): a registry of its own,
so that build functions registered for this backend do not change what nengo's reference
simulator builds, with nengo's own registry as the fallback.  Needs nengo; importing this
module without it raises ImportError (the mini-builder in `minibuilder` does not use it).
"""

import nengo.builder
from nengo.exceptions import BuildError


class Builder(nengo.builder.Builder):
    """Looks an object's build function up here first, then in nengo's registry."""

    builders = {}  # this backend's registrations only

    @classmethod
    def build(cls, model, obj, *args, **kwargs):
        generic = nengo.builder.Builder.build.__func__
        try:
            return generic(Builder, model, obj, *args, **kwargs)
        except BuildError:
            return generic(nengo.builder.Builder, model, obj, *args, **kwargs)
