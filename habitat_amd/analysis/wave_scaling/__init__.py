"""Wave scaling: the scalar strategies under the reference's names (unified,
roofline, resimplified, common, metadata), the batched entry points they are
built on (batch) and the AMD compute-unit strategy (cdna)."""
