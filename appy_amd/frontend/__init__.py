"""Front end of the annotated-loop programming model: pragma grammar,
comment-aware parsing, the decoration-time rewrite and the per-loop IR."""
