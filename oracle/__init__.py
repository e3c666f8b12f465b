"""TEST INFRASTRUCTURE -- CPU oracle of the D-NPEFF NMF hot path (see dnpeff_oracle.c)."""
