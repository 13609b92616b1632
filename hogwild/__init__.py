"""Import path of the reference package (python/hogwild/): `from hogwild.attention import hogwild_fused, ...` keeps
working for an unchanged caller.  Everything here is a re-export of `inference_lib_amd`, the MI355X implementation."""
