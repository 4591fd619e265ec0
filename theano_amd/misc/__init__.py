"""Stand-alone timing scripts for the elementwise path (the role of ``theano/misc``)."""
