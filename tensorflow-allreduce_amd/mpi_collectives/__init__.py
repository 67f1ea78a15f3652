"""MI355X-native ring collectives with the API of tensorflow.contrib.mpi_collectives."""
